"""GPU parity: every op through the C ABI (libapk_hip.so) against the CPU oracle on
the same seeded inputs.

Bars (stated per test):
  * embedding dequant+gather, router ids, grouping tables, gathers: BIT-EXACT;
  * f32 activations: max relative error <= 1e-5 (util.rel_err_f32) and the
    reference's own idiom |a-b| < 1e-5(1+|b|);
  * fp16 activations: <= 2 ulp of fp16.
Full-size cases that the oracle cannot finish in seconds are covered through
size-independent properties (row-subset equality, permutation invariants).
"""
import numpy as np
import pytest

from util import close_idiom, f16_ulp_diff, rel_err_f32, rel_err_strict

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

TOL_F32 = 1e-5
TOL_F16_ULP = 2


@pytest.fixture(scope="module")
def be():
    import allpaka_amd

    b = allpaka_amd.Backend(0)
    yield b
    b.close()


def dev(a):
    """numpy -> device tensor; uint16 arrays are fp16 bit patterns, uint32 become int32."""
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.float16).copy()).cuda()
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32).copy()).cuda()
    return torch.from_numpy(a.copy()).cuda()


def host(t):
    a = t.detach().cpu().numpy()
    if a.dtype == np.float16:
        return a.view(np.uint16)
    if a.dtype == np.int32:
        return a.view(np.uint32)
    return a


def synth():
    from allpaka_amd import synth as s

    return s


# ------------------------------------------------------------------ embedding
@pytest.mark.parametrize("fmt_name,n_in,vocab,t", [
    ("Q8_0", 1024, 997, 1), ("Q8_0", 1024, 997, 512), ("Q8_0", 32, 5, 7), ("Q8_0", 96, 33, 40), ("Q8_0", 4096, 64, 9),
    ("Q4K", 5120, 301, 1), ("Q4K", 5120, 301, 6), ("Q4K", 5120, 301, 300), ("Q4K", 256, 3, 5), ("Q4K", 1024, 17, 33),
])
@pytest.mark.parametrize("out_f16", [False, True])
def test_embed_rows_bit_exact(be, ora, fmt_name, n_in, vocab, t, out_f16):
    import allpaka_amd as apk

    s = synth()
    g = s.rng(0 if fmt_name == "Q8_0" else 2, n_in * 7 + vocab)
    table = (s.q8_0_table if fmt_name == "Q8_0" else s.q4_k_table)(g, vocab, n_in)
    ids = g.integers(0, vocab, size=t, dtype=np.uint32)
    ids[0] = vocab - 1  # last row: exercises the end-of-table tile
    if t > 1:
        ids[-1] = 0
    fmt = ora.FMT[fmt_name]
    want = ora.embed_rows(table, fmt, vocab, n_in, ids, out_f16=out_f16)
    qm = apk.QuantMat(be, dev(table), fmt, vocab, n_in)
    out = torch.full((t, n_in), 7.0, dtype=torch.float16 if out_f16 else torch.float32, device="cuda")
    qm.rows_into(dev(ids), out)
    got = host(out)
    assert np.array_equal(got.view(np.uint16 if out_f16 else np.uint32), want.view(np.uint16 if out_f16 else np.uint32))
    # QuantMat::row / row_into, one row, ids on the host
    r = qm.row(int(ids[0]), dtype=torch.float16 if out_f16 else torch.float32)
    assert np.array_equal(host(r), want[0])


def _lcg_bytes(n, state=0x243F6A8885A308D3):
    """The byte stream of the reference's GPU parity region (crates/allpaka-backend/tests/gpu_parity.rs:73-80)."""
    out = np.empty(n, np.uint8)
    mul, inc, mask = 6364136223846793005, 1442695040888963407, (1 << 64) - 1
    for i in range(n):
        state = (state * mul + inc) & mask
        out[i] = state >> 56
    return out


_SCALE_OFFS = {"Q8_0": (34, [0]), "Q2K": (84, [80, 82]), "Q3K": (110, [108]), "Q4K": (144, [0, 2]), "Q5K": (176, [0, 2]),
               "Q6K": (210, [208]), "Q5_0": (22, [0])}


@pytest.mark.parametrize("fmt_name", ["Q4K", "Q5K", "Q6K", "Q8_0", "Q2K", "Q3K", "Q5_0", "F16", "F32", "BF16"])
@pytest.mark.parametrize("out_f16", [False, True])
def test_embed_all_ten_formats_bit_exact(be, ora, fmt_name, out_f16):
    """All ten formats, hidden 512, 6 rows, the reference's fixture style: LCG bytes with the f16
    scale fields tamed to 0x211F (gpu_parity.rs:100-137, :1147-1214) -- here bit-exact, not 1e-4."""
    import allpaka_amd as apk

    fmt, hidden, vocab = ora.FMT[fmt_name], 512, 6
    rb = ora.expected_bytes(fmt, hidden)
    raw = _lcg_bytes(vocab * rb, 0x243F6A8885A308D3 + fmt)
    if fmt_name in _SCALE_OFFS:
        bb, offs = _SCALE_OFFS[fmt_name]
        blocks = raw.reshape(-1, bb)
        for o in offs:
            blocks[:, o], blocks[:, o + 1] = 0x1F, 0x21
        blocks[0, offs[0]:offs[0] + 2] = [0x01, 0x00]  # one f16-subnormal scale
    elif fmt_name == "F32":
        raw = ((np.arange(vocab * hidden) % 61 - 30) * np.float32(0.03)).astype(np.float32).view(np.uint8)
    else:  # F16 / BF16: keep the exponent away from inf/NaN so equality is meaningful
        w = raw.view(np.uint16)
        w &= np.uint16(0xBFFF)
    ids = np.array([3, 0, 5, 5, 1, 2, 4], np.uint32)
    want = ora.embed_rows(raw, fmt, vocab, hidden, ids, out_f16=out_f16)
    qm = apk.QuantMat(be, dev(raw), fmt, vocab, hidden)
    out = torch.zeros((ids.size, hidden), dtype=torch.float16 if out_f16 else torch.float32, device="cuda")
    qm.rows_into(dev(ids), out)
    got = host(out)
    assert np.array_equal(got.view(np.uint16 if out_f16 else np.uint32), want.view(np.uint16 if out_f16 else np.uint32))
    assert np.array_equal(host(qm.row(3, dtype=out.dtype)), want[0])  # token 3 of 6, as the reference's test
    # a range of rows without an id list (the dequant of a weight matrix ahead of a dense GEMM): the same rows
    want_r = ora.embed_rows(raw, fmt, vocab, hidden, np.arange(1, 6, dtype=np.uint32), out_f16=out_f16)
    got_r = host(qm.dequant_rows(1, 5, dtype=out.dtype))
    assert np.array_equal(got_r.view(np.uint16 if out_f16 else np.uint32), want_r.view(np.uint16 if out_f16 else np.uint32))
    assert qm.dequant_rows(6, 0, dtype=out.dtype).shape == (0, hidden)
    with pytest.raises(apk.Declined):
        qm.dequant_rows(2, 5)  # rows 2..6 of 6
    # models that scale their token embeddings: one f32 multiply after the dequant (prefill.rs:107-109;
    # Gemma's factor is sqrt(hidden), here of a 3584-wide model)
    scale = float(np.sqrt(np.float32(3584.0)))
    want_s = ora.embed_rows(raw, fmt, vocab, hidden, ids, out_f16=out_f16, scale=scale)
    assert not np.array_equal(want_s, want)
    qm.rows_into(dev(ids), out, embed_scale=scale)
    got = host(out)
    assert np.array_equal(got.view(np.uint16 if out_f16 else np.uint32), want_s.view(np.uint16 if out_f16 else np.uint32))


@pytest.mark.parametrize("fmt_name,n_in", [("Q8_0", 20480), ("Q6K", 12288), ("Q5K", 16384), ("Q2K", 9216), ("Q3K", 8448),
                                           ("Q5_0", 9984), ("F32", 4104), ("Q4K", 16384), ("BF16", 32752)])
@pytest.mark.parametrize("out_f16", [False, True])
def test_embed_long_rows_take_several_workgroups(be, ora, fmt_name, n_in, out_f16):
    """Rows longer than one workgroup covers (chunks of a row), up to the staging limit of the LDS-staged formats."""
    import allpaka_amd as apk

    fmt, vocab = ora.FMT[fmt_name], 5
    g = np.random.default_rng(n_in)
    rb = ora.expected_bytes(fmt, n_in)
    raw = g.integers(0, 256, size=vocab * rb, dtype=np.uint8)
    if fmt_name in _SCALE_OFFS:
        bb, offs = _SCALE_OFFS[fmt_name]
        blocks = raw.reshape(-1, bb)
        for o in offs:
            blocks[:, o + 1] &= 0x3B  # finite, small f16 scale fields
    elif fmt_name == "F32":
        raw = synth().normal_f32(g, vocab * n_in).view(np.uint8).copy()
    else:
        raw.view(np.uint16)[:] &= np.uint16(0xBFFF)
    ids = np.array([4, 0, 2, 4], np.uint32)
    want = ora.embed_rows(raw, fmt, vocab, n_in, ids, out_f16=out_f16)
    qm = apk.QuantMat(be, dev(raw), fmt, vocab, n_in)
    out = torch.zeros((ids.size, n_in), dtype=torch.float16 if out_f16 else torch.float32, device="cuda")
    qm.rows_into(dev(ids), out)
    v = np.uint16 if out_f16 else np.uint32
    assert np.array_equal(host(out).view(v), want.view(v))


@pytest.mark.parametrize("fmt_name", ["Q4K", "Q5K", "Q6K", "Q8_0", "Q2K", "Q3K", "Q5_0", "F16", "F32", "BF16"])
@pytest.mark.parametrize("hidden", [512, 1280])
def test_embed_device_ids_out_of_vocab_leave_their_rows_and_raise_the_flag(be, ora, fmt_name, hidden):
    """Ids that live on the device cannot be checked before the launch: a row whose id is >= vocab is left as it
    was, its neighbours (which may share a wave, a workgroup or neither with it) are gathered as usual, and the
    status word reports it once read -- for every format's kernel, fp16 and f32 output."""
    fmt, vocab = ora.FMT[fmt_name], 9
    g = np.random.default_rng(hidden + fmt)
    rb = ora.expected_bytes(fmt, hidden)
    raw = g.integers(0, 256, size=vocab * rb, dtype=np.uint8)
    if fmt_name in _SCALE_OFFS:
        bb, offs = _SCALE_OFFS[fmt_name]
        for o in offs:
            raw.reshape(-1, bb)[:, o + 1] &= 0x3B  # finite, small f16 scale fields
    elif fmt_name == "F32":
        raw = synth().normal_f32(synth().rng(4, hidden), vocab * hidden).view(np.uint8).copy()
    else:
        raw.view(np.uint16)[:] &= np.uint16(0xBFFF)
    table = dev(raw)
    ids = np.array([4, 9, 0, 8, 0xFFFFFFFF, 2, 2, 100, 7], np.uint32)
    good = ids < vocab
    for out_f16 in (False, True):
        want = ora.embed_rows(raw, fmt, vocab, hidden, np.where(good, ids, 0).astype(np.uint32), out_f16=out_f16)
        out = torch.full((ids.size, hidden), 3.0, dtype=torch.float16 if out_f16 else torch.float32, device="cuda")
        assert be.take_faults() == 0
        rc = be.L.apk_embed_rows(be.h, fmt, table.data_ptr(), vocab, hidden, dev(ids).data_ptr(), ids.size, out.data_ptr(),
                                 1 if out_f16 else 0)
        assert rc == 0
        got = host(out)
        v = np.uint16 if out_f16 else np.uint32
        assert np.array_equal(got[good].view(v), want[good].view(v))
        assert np.all(got[~good].view(v) == (0x4200 if out_f16 else 0x40400000))  # still 3.0
        assert be.take_faults() & 1 and be.take_faults() == 0  # APK_FAULT_TOKEN_RANGE, cleared by the read


def test_embed_subnormal_scales_and_reference_vectors(be, ora):
    import allpaka_amd as apk

    # the reference's Q8_0 known answer (dequant.rs:317-331) and a block of f16-subnormal scales
    block = np.zeros((4, 34), np.uint8)
    block[0, 0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    block[0, 2], block[0, 3], block[0, 33] = 10, np.uint8(236), 127
    for r, code in enumerate([0x0001, 0x03FF, 0x8001], start=1):
        block[r, 0:2] = np.frombuffer(np.uint16(code).tobytes(), np.uint8)
        block[r, 2:] = np.arange(-16, 16, dtype=np.int8).view(np.uint8) * 7
    qm = apk.QuantMat(be, dev(block.reshape(-1)), ora.FMT["Q8_0"], 4, 32)
    out = torch.zeros((4, 32), dtype=torch.float32, device="cuda")
    qm.rows_into(dev(np.arange(4, dtype=np.uint32)), out)
    got = host(out)
    assert got[0, 0] == 5.0 and got[0, 1] == -10.0 and got[0, 31] == 63.5 and got[0, 2] == 0.0
    want = ora.embed_rows(block.reshape(-1), ora.FMT["Q8_0"], 4, 32, np.arange(4, dtype=np.uint32))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert got[1, 0] == np.float32(-112 * 2.0 ** -24)
    # Q4_K known answer (dequant.rs:448-468)
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blk[2:4] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blk[4], blk[5], blk[8], blk[9], blk[16] = 2, 3, 1, 2, 0x75
    qm = apk.QuantMat(be, dev(blk), ora.FMT["Q4K"], 1, 256)
    got = host(qm.row(0))
    assert got[0] == 9.0 and got[1] == -1.0 and got[32] == 19.0 and got[33] == -2.0 and np.all(got[64:] == 0.0)


def test_embed_with_the_ids_on_the_host(be, ora):
    """apk_embed_rows_host_ids: the ids are range-checked before anything is enqueued (as the reference's
    callers reject token >= vocab first); a single token travels as a kernel argument, more through a pinned
    staging buffer -- the same rows as the device-id entry either way, call after call."""
    import ctypes as C

    import allpaka_amd.lib as apklib

    s = synth()
    vocab, hidden = 300, 512
    for fmt_name in ("Q4K", "Q8_0", "F16"):
        fmt = ora.FMT[fmt_name]
        rb = ora.expected_bytes(fmt, hidden)
        raw = _lcg_bytes(vocab * rb, 0x9E3779B97F4A7C15 + fmt)
        if fmt_name in _SCALE_OFFS:
            bb, offs = _SCALE_OFFS[fmt_name]
            for o in offs:
                raw.reshape(-1, bb)[:, o], raw.reshape(-1, bb)[:, o + 1] = 0x1F, 0x21
        else:
            raw.view(np.uint16)[:] &= np.uint16(0xBFFF)
        table = dev(raw)
        for ids in ([7], [299], [5, 0, 299, 5, 17], list(range(40, 90)), [3]):
            want = ora.embed_rows(raw, fmt, vocab, hidden, np.array(ids, np.uint32), out_f16=True)
            out = torch.zeros((len(ids), hidden), dtype=torch.float16, device="cuda")
            harr = (C.c_uint32 * len(ids))(*ids)
            apklib.check(be.L.apk_embed_rows_host_ids(be.h, fmt, table.data_ptr(), vocab, hidden, harr, len(ids), out.data_ptr(), apklib.F16))
            be.sync()
            assert np.array_equal(host(out), want), (fmt_name, ids)
        for bad in ([300], [1, 2, 300]):
            harr = (C.c_uint32 * len(bad))(*bad)
            out = torch.full((len(bad), hidden), 2.0, dtype=torch.float16, device="cuda")
            rc = be.L.apk_embed_rows_host_ids(be.h, fmt, table.data_ptr(), vocab, hidden, harr, len(bad), out.data_ptr(), apklib.F16)
            be.sync()
            assert rc == apklib.DECLINE_RANGE and torch.all(out == 2.0) and be.take_faults() == 0


def test_embed_errors_and_declines(be, ora):
    import allpaka_amd as apk

    data = dev(np.zeros(34 * 2, np.uint8))
    qm = apk.QuantMat(be, data, ora.FMT["Q8_0"], 1, 64)
    with pytest.raises(ValueError):  # quantmat/mod.rs:923-937: row(1) of a 1-row matrix
        qm.row(1)
    with pytest.raises(ValueError):
        apk.QuantMat(be, data, ora.FMT["Q8_0"], 1, 48)
    with pytest.raises(ValueError):
        apk.QuantMat(be, data[:-1], ora.FMT["Q8_0"], 1, 64)
    with pytest.raises(ValueError):
        qm.row_into(0, torch.zeros(32, device="cuda"))
    # device-side ids out of vocab: no fault, the row is left untouched, the status word says so
    out = torch.full((2, 64), 3.0, device="cuda")
    with pytest.raises(ValueError):
        qm.rows_into(dev(np.array([0, 5], np.uint32)), out)
    assert np.all(host(out)[1] == 3.0) and np.all(host(out)[0] == 0.0)
    assert be.take_faults() == 0  # cleared by the read above
    # a row the device path does not take (not whole 16-byte output tiles) declines, it does not fail
    f32m = apk.QuantMat(be, dev(np.zeros(12, np.uint8)), ora.FMT["F32"], 1, 3)
    with pytest.raises(apk.Declined):
        f32m.row(0)
    with pytest.raises(ValueError):
        apk.QuantMat(be, data, 42, 1, 64)


# ------------------------------------------------------------- add + RMSNorm
@pytest.mark.parametrize("n,rows", [(1024, 1), (1024, 512), (5120, 1), (5120, 6), (5120, 64), (2048, 33), (128, 5),
                                    (8, 3), (4096 + 64, 3), (8192, 2), (16384, 2),
                                    # short rows in bulk: several rows per wave
                                    (128, 100), (8, 33), (256, 77), (64, 1000), (24, 16), (200, 19), (104, 4097),
                                    # batches beyond one resident round of waves: two tiles per lane, several waves per row
                                    (5120, 4100), (4096, 2100), (16384, 1030), (1032, 4100), (8192, 520), (2560, 8200)])
@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("with_delta", [True, False])
def test_add_rmsnorm_rows(be, ora, n, rows, f16, with_delta):
    s = synth()
    g = s.rng(1, n + rows)
    x = s.normal_f32(g, (rows, n))
    d = s.normal_f32(g, (rows, n))
    gamma = s.normal_f32(g, n, 1.0, 0.05)
    if f16:
        x, d = s.to_f16_bits(x), s.to_f16_bits(d)
    wx, wh = x.copy(), np.zeros_like(x)
    ora.add_rmsnorm_rows(wx, d if with_delta else None, wh, gamma, 1e-6)
    tx, th = dev(x), torch.zeros_like(dev(x))
    be.add_rmsnorm_rows(tx, dev(d) if with_delta else None, th, dev(gamma), 1e-6)
    gx, gh = host(tx), host(th)
    if f16:
        assert np.array_equal(gx, wx)  # the residual sum rounds once: bit-exact
        assert f16_ulp_diff(gh, wh) <= TOL_F16_ULP
    else:
        assert np.array_equal(gx, wx)  # f32 add is exact-same
        assert rel_err_f32(gh, wh) <= TOL_F32 and close_idiom(gh, wh)
        assert np.mean(gh.view(np.uint32) == wh.view(np.uint32)) > 0.999  # f64 statistics: bit-equal almost everywhere


@pytest.mark.parametrize("n,rows", [(2304, 1), (3584, 6), (1152, 64), (2560, 300), (3840, 2100), (5376, 700), (2560, 4200), (1024, 9000),
                                    (8192, 3), (16384, 2),
                                    # more fp16 rows than are resident at once: 5, 3 and 4 tiles per lane, 2 or 3 waves per row
                                    (5120, 3100), (4608, 3100), (3584, 3100),
                                    # outside the tiled kernels: the two steps run
                                    (1001, 5), (64, 100), (20488, 2)])
@pytest.mark.parametrize("f16", [False, True])
def test_postnorm_add_rmsnorm_rows(be, ora, n, rows, f16):
    """The sandwich norm of the Gemma family and the next norm in one pass (decode.rs:581-584, :771-775, :762-764):
    x += rmsnorm(delta) * post_gamma; h = rmsnorm(x) * gamma -- against the oracle's three ops in the reference's order."""
    s = synth()
    g = s.rng(1, n * 3 + rows)
    x, d = s.normal_f32(g, (rows, n)), s.normal_f32(g, (rows, n), 0.0, 3.0)
    pg, gamma = s.normal_f32(g, n, 1.0, 0.05), s.normal_f32(g, n, 1.0, 0.05)
    if f16:
        x, d = s.to_f16_bits(x), s.to_f16_bits(d)
    nd = np.zeros_like(d)
    ora.add_rmsnorm_rows(d.copy(), None, nd, pg, 1e-6)  # ops::rmsnorm(projected, post_norm, eps)
    wx, wh = x.copy(), np.zeros_like(x)
    ora.add_rmsnorm_rows(wx, nd, wh, gamma, 1e-6)       # add_assign_slice, then rmsnorm_into
    tx, td, th = dev(x), dev(d), torch.zeros_like(dev(x))
    be.postnorm_add_rmsnorm_rows(tx, td, dev(pg), th, dev(gamma), 1e-6)
    gx, gh = host(tx), host(th)
    if f16:
        # one launch: the normalised delta is the reference's f32 value rounded once, so the sum is the oracle's bit for
        # bit; as two steps the first is the plain fp16 row norm (1 ulp of the normalised delta in rare elements, which
        # a cancelling sum magnifies): there the sum is held to 1 ulp of its larger operand
        import allpaka_amd.lib as apklib

        p = apklib.Plan()
        assert be.L.apk_plan_postnorm_add_rmsnorm_rows(n, rows, 1, p) == 0
        if p.kernel.startswith(b"apk_postnorm"):
            assert np.array_equal(gx, wx)
        else:
            fv = lambda a: a.view(np.float16).astype(np.float64)  # noqa: E731
            key = lambda b: np.where(b.astype(np.int32) & 0x8000, 0x8000 - b.astype(np.int32), b.astype(np.int32))  # noqa: E731
            slack = 2.0 ** -10 * np.maximum(np.abs(fv(x)), np.abs(fv(nd)))
            assert np.all((np.abs(key(gx) - key(wx)) <= TOL_F16_ULP) | (np.abs(fv(gx) - fv(wx)) <= slack))
            assert np.mean(gx == wx) > 0.999
        assert f16_ulp_diff(gh, wh) <= TOL_F16_ULP or not p.kernel.startswith(b"apk_postnorm")
    else:
        assert rel_err_f32(gx, wx) <= TOL_F32 and close_idiom(gx, wx)
        assert rel_err_f32(gh, wh) <= TOL_F32 and close_idiom(gh, wh)
        assert np.mean(gx.view(np.uint32) == wx.view(np.uint32)) > 0.999  # f64 statistics: bit-equal almost everywhere
    import allpaka_amd as apk

    with pytest.raises(apk.Declined):  # x, delta and h must be three tensors
        be.postnorm_add_rmsnorm_rows(tx, tx, dev(pg), th, dev(gamma), 1e-6)


def test_rmsnorm_reference_vectors_and_asserts(be, ora):
    # ops/mod.rs:119-144, :412-419
    x = torch.tensor([3.0, -4.0, 12.0, 0.0], device="cuda")
    be.rmsnorm(x, torch.ones(4, device="cuda"), 0.0)
    h = host(x)
    assert abs(float(np.sqrt((h * h).sum() / 4)) - 1.0) < 1e-5 and h[0] > 0 and h[1] < 0 and h[3] == 0
    x = torch.zeros(8, device="cuda")
    be.rmsnorm(x, torch.ones(8, device="cuda"), 1e-5)
    assert np.all(np.isfinite(host(x)))
    with pytest.raises(AssertionError, match="dst holds fewer rows than src"):
        be.rmsnorm_rows_into(torch.zeros(8 * 1024, device="cuda"), torch.ones(64 * 1024, device="cuda"),
                             torch.ones(1024, device="cuda"), 1e-6)
    with pytest.raises(AssertionError):
        be.rmsnorm(torch.zeros(4, device="cuda"), torch.zeros(8, device="cuda"), 0.0)
    import allpaka_amd as apk

    with pytest.raises(apk.Declined):  # a norm written over its own input while a residual is added: declined
        t6 = torch.zeros(6, device="cuda")
        be.add_rmsnorm_rows(t6, t6.clone(), t6, torch.ones(6, device="cuda"), 0.0)
    # rows of any length take the element-wise path: ops/mod.rs:130-135 ([1,1] * [2,3]), odd lengths, and
    # rows longer than the tiled kernels hold (beyond 20 480 elements), for both activation types
    x = torch.tensor([1.0, 1.0], device="cuda")
    be.rmsnorm(x, torch.tensor([2.0, 3.0], device="cuda"), 0.0)
    assert abs(host(x)[0] - 2.0) < 1e-5 and abs(host(x)[1] - 3.0) < 1e-5
    for rows, n in [(2, 6), (3, 1031), (2, 32768), (1, 40001)]:
        g = synth().rng(1, n + 1)
        xs, ds = synth().to_f16_bits(synth().normal_f32(g, (rows, n))), synth().to_f16_bits(synth().normal_f32(g, (rows, n)))
        gm = synth().normal_f32(g, n, 1.0, 0.05)
        wx, wh = xs.copy(), np.zeros_like(xs)
        ora.add_rmsnorm_rows(wx, ds, wh, gm, 1e-6)
        tx, th = dev(xs), torch.zeros_like(dev(xs))
        be.add_rmsnorm_rows(tx, dev(ds), th, dev(gm), 1e-6)
        assert np.array_equal(host(tx), wx) and f16_ulp_diff(host(th), wh) <= TOL_F16_ULP, (rows, n)
    for rows, n in [(1, 6), (5, 1031), (3, 7), (2, 40004)]:
        g = synth().rng(1, n)
        xs, ds = synth().normal_f32(g, (rows, n)), synth().normal_f32(g, (rows, n))
        gm = synth().normal_f32(g, n, 1.0, 0.05)
        wx, wh = xs.copy(), np.zeros_like(xs)
        ora.add_rmsnorm_rows(wx, ds, wh, gm, 1e-6)
        tx, th = dev(xs), torch.zeros_like(dev(xs))
        be.add_rmsnorm_rows(tx, dev(ds), th, dev(gm), 1e-6)
        assert np.array_equal(host(tx), wx) and rel_err_f32(host(th), wh) <= TOL_F32
    src = torch.randn(40, 1024, device="cuda")
    w = torch.randn(1024, device="cuda")
    dst = torch.zeros_like(src)
    be.rmsnorm_rows_into(dst, src, w, 1e-6)
    want = np.zeros((40, 1024), np.float32)
    ora.rmsnorm_rows_into(want, host(src), host(w), 1e-6, threads=4)
    assert rel_err_f32(host(dst), want) <= TOL_F32


# ------------------------------------------------------- QK-norm + NeoX RoPE
def _qk_case(ora, cfg, rows, n_q, n_kv, hd, f16, positions, theta=1e6):
    s = synth()
    g = s.rng(cfg, rows * 131 + n_q)
    q = s.normal_f32(g, (rows, n_q * hd))
    k = s.normal_f32(g, (rows, n_kv * hd))
    qw = s.normal_f32(g, hd, 1.0, 0.05)
    kw = s.normal_f32(g, hd, 1.0, 0.05)
    if f16:
        q, k = s.to_f16_bits(q), s.to_f16_bits(k)
    inv = ora.rope_inv_freq(hd, theta)
    ropes = ora.rope_table(positions, inv)
    return q, k, qw, kw, inv, ropes


@pytest.mark.parametrize("rows,n_q,n_kv,hd,pos_kind", [
    (1, 16, 8, 128, "one"), (512, 16, 8, 128, "prefill"), (1, 64, 8, 128, "one"), (6, 64, 8, 128, "verify"),
    (64, 64, 8, 128, "multi"), (5, 3, 1, 64, "multi"), (3, 2, 2, 256, "multi"), (7, 1, 0, 128, "multi"),
])
@pytest.mark.parametrize("f16", [False, True])
def test_qknorm_rope(be, ora, rows, n_q, n_kv, hd, pos_kind, f16):
    g = synth().rng(3, rows)
    positions = {"one": [int(g.integers(0, 4096))], "prefill": list(range(rows)), "verify": list(range(1000, 1000 + rows)),
                 "multi": [int(p) for p in g.integers(0, 32768, size=rows)]}[pos_kind]
    q, k, qw, kw, inv, ropes = _qk_case(ora, 3, rows, n_q, n_kv, hd, f16, positions)
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6)
    tq, tk = dev(q), dev(k)
    be.qknorm_rope_neox(tq, tk, dev(qw), dev(kw), dev(ropes), n_q, n_kv, hd, 1e-6)
    for got, want in ((host(tq), wq), (host(tk), wk)):
        if f16:
            assert f16_ulp_diff(got, want) <= TOL_F16_ULP
        else:
            assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want)
            # without a floor: strictly element by element wherever the output has not cancelled ...
            assert rel_err_strict(got, want) <= TOL_F32
            # ... and EVERY element, cancelled or not, against the size of the pair it was rotated from (a rotation keeps
            # a pair's length, so that is sqrt(w[i]^2 + w[i + hd/2]^2) of the expected outputs): a few f32 ulps of it,
            # which is all that inputs of that size can carry -- forty times tighter than 1e-5
            if want.size:
                w4 = want.astype(np.float64).reshape(rows, -1, 2, hd // 2)
                g4 = got.astype(np.float64).reshape(rows, -1, 2, hd // 2)
                pair = np.sqrt(w4[:, :, 0] ** 2 + w4[:, :, 1] ** 2)[:, :, None, :]
                assert np.all(np.abs(g4 - w4) <= 4 * 2.0 ** -24 * pair + 1e-37)


@pytest.mark.parametrize("scale", [1.0, 100.0, 1e-3])
def test_qknorm_rope_fp16_is_the_reference_result_rounded_once(be, ora, scale):
    """A rotated output a*cos - b*sin can nearly cancel, and an f32-level difference is then many fp16 ulps: the
    per-head norm in front of the rotation therefore reproduces the reference's f32 values (f64 statistics, the
    f64 product rounded to f32, uncontracted rotation), and the fp16 result is that value rounded once --
    bit for bit on these 900 000 elements, many of them in the cancellation zone."""
    s = synth()
    g = s.rng(3, int(scale * 1000) + 77)
    rows, n_q, n_kv, hd = 96, 64, 8, 128
    q = s.to_f16_bits(s.normal_f32(g, (rows, n_q * hd)) * np.float32(scale))
    k = s.to_f16_bits(s.normal_f32(g, (rows, n_kv * hd)) * np.float32(scale))
    qw, kw = s.normal_f32(g, hd, 1.0, 0.05), s.normal_f32(g, hd, 1.0, 0.05)
    ropes = ora.rope_table([int(v) for v in g.integers(0, 32768, size=rows)], ora.rope_inv_freq(hd, 1e6))
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6)
    tq, tk = dev(q), dev(k)
    be.qknorm_rope_neox(tq, tk, dev(qw), dev(kw), dev(ropes), n_q, n_kv, hd, 1e-6)
    assert np.array_equal(host(tq), wq) and np.array_equal(host(tk), wk)


def test_rope_only_and_reference_vectors(be, ora):
    # no norm weights: rotation only (attention.rs:140-146); bit-exact (same f32 ops, no contraction)
    rows, n_q, n_kv, hd = 9, 4, 2, 128
    positions = [0, 1, 17, 5000, 4097, 32767, 3, 511, 12345]
    q, k, _, _, inv, ropes = _qk_case(ora, 3, rows, n_q, n_kv, hd, False, positions)
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, None, None, ropes, 1e-6)
    tq, tk = dev(q), dev(k)
    be.qknorm_rope_neox(tq, tk, None, None, dev(ropes), n_q, n_kv, hd, 1e-6)
    assert np.array_equal(host(tq), wq) and np.array_equal(host(tk), wk)
    assert np.array_equal(host(tq)[0], q[0])  # position 0 is the identity (ops/mod.rs:188-202)
    # pairing: a one-hot channel 0 moves energy to channel hd/2 (ops/mod.rs:206-221)
    x = torch.zeros(128, device="cuda")
    x[0] = 1.0
    t1 = ora.rope_sin_cos(1, ora.rope_inv_freq(128, 10000.0))
    be.rope_neox_cached_from_array(x, dev(t1))
    h = host(x)
    assert abs(h[64] - np.sin(np.float32(1.0))) < 1e-6 and h[1] == 0.0
    import allpaka_amd as apk

    tr = dev(ropes)
    for bad_hd, bad_rot in ((128, 63), (64, 128), (0, 0)):  # odd rotary width; wider than the head; no head
        rc = be.L.apk_qknorm_rope_neox(be.h, tq.data_ptr(), tk.data_ptr(), None, None, tr.data_ptr(), 2, n_q, n_kv, bad_hd, bad_rot,
                                       1e-6, apk.lib.F32)
        assert rc == apk.lib.DECLINE_SHAPE, (bad_hd, bad_rot)
    be.sync()
    assert np.array_equal(host(tq), wq)  # declined: nothing touched
    # adjacent-pair style: a one-hot channel 0 moves energy to channel 1 (rope.rs:90-101)
    x = torch.zeros(128, device="cuda")
    x[0] = 1.0
    be.rope_norm_cached_from_array(x, dev(t1))
    h = host(x)
    assert abs(h[1] - np.sin(np.float32(1.0))) < 1e-6 and h[64] == 0.0
    # the reference's partial-rotary vector: a 12-wide head rotating its first 8 channels (ops/mod.rs:367-391)
    inv4 = ora.rope_inv_freq(8, 10000.0)
    t4 = ora.rope_sin_cos(5, inv4)
    for name in ("rope_neox_cached_from_array", "rope_norm_cached_from_array"):
        a = (np.arange(12, dtype=np.float32) * 0.25 - 1.0).astype(np.float32)
        want = a.copy()
        getattr(ora, name)(want, t4)
        ta = dev(a)
        getattr(be, name)(ta, dev(t4))
        assert np.array_equal(host(ta), want)
        assert np.array_equal(want[8:], a[8:])  # the tail passes through


@pytest.mark.parametrize("rows,n_q,n_kv,hd,rot", [
    (5, 4, 2, 128, 64),   # partial rotary on a tiled head size (GLM style)
    (3, 6, 2, 96, 96), (7, 5, 1, 80, 32), (2, 2, 2, 192, 192), (4, 3, 3, 32, 16), (1, 1, 1, 576, 64), (3, 2, 1, 128, 0),
    # partial rotary over heads of 64 / 128 / 256: the tiled kernels where the rotary width is whole tiles, one and
    # two passes per q wave; (128, 8) is whole tiles only for some of the style / type combinations
    (300, 32, 8, 128, 64), (9, 8, 2, 256, 64), (33, 12, 2, 64, 32), (7, 4, 4, 128, 32), (5, 4, 2, 128, 96), (4, 3, 1, 128, 8),
    (6, 2, 2, 64, 48), (700, 16, 2, 256, 128), (40, 20, 0, 128, 16),
])
@pytest.mark.parametrize("style", [0, 1])
@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("normed", [True, False])
def test_qknorm_rope_any_geometry(be, ora, rows, n_q, n_kv, hd, rot, style, f16, normed):
    """Head sizes outside 64/128/256, partial rotary and the adjacent-pair style: the reference's caller loop
    (attention.rs:131-165 with rope_from_arrays :62-67) through the element-wise kernel."""
    s = synth()
    g = s.rng(3, rows * 977 + hd * 13 + rot + style)
    q, k = s.normal_f32(g, (rows, n_q * hd)), s.normal_f32(g, (rows, n_kv * hd))
    qw, kw = (s.normal_f32(g, hd, 1.0, 0.05), s.normal_f32(g, hd, 1.0, 0.05)) if normed else (None, None)
    if f16:
        q, k = s.to_f16_bits(q), s.to_f16_bits(k)
    positions = [int(v) for v in g.integers(0, 32768, size=rows)]
    if rot:
        ropes = ora.rope_table(positions, ora.rope_inv_freq(rot, 1e6))
    else:
        ropes = np.zeros((rows, 0, 2), np.float32)
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6, style=style)
    tq, tk = dev(q), dev(k)
    fn = be.qknorm_rope_norm if style else be.qknorm_rope_neox
    rt = dev(ropes) if rot else torch.zeros((rows, 0, 2), device="cuda")
    fn(tq, tk, None if qw is None else dev(qw), None if kw is None else dev(kw), rt, n_q, n_kv, hd, 1e-6, rot_dim=rot)
    for got, want in ((host(tq), wq), (host(tk), wk)):
        if f16:
            assert f16_ulp_diff(got, want) <= TOL_F16_ULP
        elif not normed:
            assert np.array_equal(got, want)  # rotation only: the same f32 operations
        else:
            assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want)


@pytest.mark.parametrize("rows,n_q,n_kv,hd", [(1, 32, 8, 128), (6, 32, 8, 128), (64, 32, 8, 128), (300, 32, 8, 128), (2048, 8, 2, 128),
                                            (700, 64, 8, 128), (33, 12, 2, 64), (400, 32, 8, 64), (9, 8, 1, 256), (350, 16, 4, 256),
                                            (5, 3, 0, 128), (5, 0, 3, 64)])
@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("normed", [True, False])
def test_adjacent_pair_rope_on_whole_heads(be, ora, rows, n_q, n_kv, hd, f16, normed):
    """RopeStyle::Norm (pairs (2i, 2i+1), rope.rs:52-64: the Llama-family layout, attention.rs:62-67) over whole
    heads of 64 / 128 / 256: the tiled kernels, one and two passes per q wave, with and without the QK-norm."""
    s = synth()
    g = s.rng(3, rows * 131 + n_q * 7 + hd)
    q, k = s.normal_f32(g, (rows, n_q * hd)), s.normal_f32(g, (rows, n_kv * hd))
    qw, kw = (s.normal_f32(g, hd, 1.0, 0.05), s.normal_f32(g, hd, 1.0, 0.05)) if normed else (None, None)
    if f16:
        q, k = s.to_f16_bits(q), s.to_f16_bits(k)
    ropes = ora.rope_table([int(v) for v in g.integers(0, 32768, size=rows)], ora.rope_inv_freq(hd, 5e5))
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-5, style=1)
    tq, tk = dev(q), dev(k)
    be.qknorm_rope_norm(tq, tk, None if qw is None else dev(qw), None if kw is None else dev(kw), dev(ropes), n_q, n_kv, hd, 1e-5)
    for got, want in ((host(tq), wq), (host(tk), wk)):
        if f16:
            assert np.array_equal(got, want)  # the definition, bit for bit (as the NeoX kernels)
        elif not normed:
            assert np.array_equal(got, want)  # rotation only: the same f32 operations
        else:
            assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want)


def test_rope_table_on_device(be, ora):
    # table rows built on the device vs ops::rope_sin_cos: same f32 angle, device sincosf vs glibc
    inv = ora.rope_inv_freq(128, 1e6)
    g = synth().rng(3, 99)
    positions = np.concatenate([np.arange(0, 512), g.integers(0, 32768, size=64)]).astype(np.uint32)
    want = ora.rope_table(positions, inv)
    got = host(be.rope_table(dev(positions), dev(inv)))
    # the device rounds the double-precision sine/cosine of the same f32 angle once: the correctly rounded
    # value, which glibc returns in all but rare cases -- bit-equal almost everywhere, 1 ulp at worst
    assert np.max(np.abs(got - want)) <= 6e-8
    assert np.mean(got.view(np.uint32) == want.view(np.uint32)) > 0.98  # glibc sinf/cosf: 0.56 ulp, ~1 % off by one
    # and used end to end on the 64 long-context rows (fp16 config)
    rows, n_q, n_kv, hd = 64, 64, 8, 128
    q, k, qw, kw, _, ropes = _qk_case(ora, 3, rows, n_q, n_kv, hd, True, positions[512:])
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6)
    tq, tk = dev(q), dev(k)
    be.qknorm_rope_neox(tq, tk, dev(qw), dev(kw), be.rope_table(dev(positions[512:].copy()), dev(inv)), n_q, n_kv, hd, 1e-6)
    assert f16_ulp_diff(host(tq), wq) <= TOL_F16_ULP and f16_ulp_diff(host(tk), wk) <= TOL_F16_ULP


# --------------------------------------------- fused K/V cache store
@pytest.mark.parametrize("rows,n_q,n_kv,hd,f16", [(1, 16, 8, 128, False), (64, 64, 8, 128, True), (300, 64, 8, 128, True),
                                                   (7, 4, 4, 64, False), (5, 2, 1, 256, True), (2048, 16, 8, 128, False)])
@pytest.mark.parametrize("style", [0, 1])
@pytest.mark.parametrize("partial", [False, True])
def test_qknorm_rope_kv_store(be, ora, rows, n_q, n_kv, hd, f16, style, partial):
    """QK-norm + RoPE with KvCache::store_at fused: q, k as the plain op; the cache rows hold
    the rotated k and the row's v narrowed to f16 (RNE) at each row's position."""
    s = synth()
    g = s.rng(3, rows * 3 + hd)
    cap = max(rows + 9, 40)
    positions = g.permutation(cap)[:rows].astype(np.uint32)  # distinct cache rows, any order
    q, k, qw, kw, inv, ropes = _qk_case(ora, 3, rows, n_q, n_kv, hd, f16, [int(p) for p in positions])
    rot = hd // 2 if partial else hd
    if partial:  # only the leading half of every head rotates
        ropes = ora.rope_table([int(p) for p in positions], ora.rope_inv_freq(rot, 1e6))
    v = s.normal_f32(g, (rows, n_kv * hd))
    if f16:
        v = s.to_f16_bits(v)
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6, style=style)
    wkc, wvc = np.zeros((cap, n_kv * hd), np.uint16), np.zeros((cap, n_kv * hd), np.uint16)
    ora.kv_store_rows(wk, v, positions, wkc, wvc)
    tq, tk = dev(q), dev(k)
    kc = torch.zeros((cap, n_kv * hd), dtype=torch.float16, device="cuda")
    vc = torch.zeros_like(kc)
    be.qknorm_rope_kv_store(tq, tk, dev(v), dev(qw), dev(kw), dev(ropes), dev(positions), kc, vc, n_q, n_kv, hd, 1e-6,
                            adjacent_pairs=bool(style), rot_dim=rot)
    gk = host(tk)
    for got, want in ((host(tq), wq), (gk, wk)):
        if f16:
            assert f16_ulp_diff(got, want) <= TOL_F16_ULP
        else:
            assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want)
    assert np.array_equal(host(vc), wvc)  # v: a pure narrowing, bit-exact
    # k cache: exactly the narrowing of the k this launch produced, and within 1 fp16 ulp (2 on the fp16 path) of the oracle's
    mine_k, mine_v = np.zeros_like(wkc), np.zeros_like(wvc)
    ora.kv_store_rows(gk, v, positions, mine_k, mine_v)
    assert np.array_equal(host(kc), mine_k)
    assert f16_ulp_diff(host(kc), wkc) <= (TOL_F16_ULP if f16 else 1)


@pytest.mark.parametrize("rows,n_q,n_kv,hd,rot,f16", [(1, 64, 8, 128, 128, True), (64, 64, 8, 128, 128, True), (6, 16, 8, 128, 128, False),
                                                       (1, 16, 8, 128, 128, False), (8, 4, 4, 64, 32, True), (5, 2, 1, 256, 256, False),
                                                       (3, 3, 2, 96, 64, False), (64, 1, 0, 128, 128, True), (2, 4, 2, 80, 0, False)])
@pytest.mark.parametrize("style", [0, 1])
@pytest.mark.parametrize("store", [False, True])
def test_qknorm_rope_with_positions_inside_the_launch(be, ora, rows, n_q, n_kv, hd, rot, f16, style, store):
    """A decode-sized batch with the rotary angles taken from the rows' positions in the kernel (no table): the oracle's
    rope_sin_cos rows on the CPU side; on the device also equal to apk_rope_table followed by the table form, bit for bit,
    wherever that form takes the same arithmetic path (heads outside 64 / 128 / 256 or a partial rotary width)."""
    import allpaka_amd as apk

    store = store and n_kv > 0  # (no k heads: nothing to store, the plain form runs twice)
    s = synth()
    g = s.rng(3, rows * 7 + hd + rot)
    cap = 40000
    positions = g.integers(0, 32768, size=rows).astype(np.uint32)
    positions[0] = 0
    q, k, qw, kw, _, _ = _qk_case(ora, 3, rows, n_q, n_kv, hd, f16, [0] * rows)
    inv = ora.rope_inv_freq(rot, 1e6) if rot else np.zeros(0, np.float32)
    ropes = ora.rope_table([int(p) for p in positions], inv) if rot else np.zeros((rows, 0, 2), np.float32)
    v = s.normal_f32(g, (rows, n_kv * hd))
    if f16:
        v = s.to_f16_bits(v)
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6, style=style)
    tq, tk = dev(q), dev(k)
    kc = vc = None
    if store:
        # a small cache addressed through a position map would hide a wrong row: the cache is as long as the context
        kc = torch.zeros((cap, n_kv * hd), dtype=torch.float16, device="cuda")
        vc = torch.zeros_like(kc)
    d0 = be.stats()[1]
    be.qknorm_rope_pos(tq, tk, dev(qw), dev(kw), dev(positions), dev(inv) if rot else torch.zeros(1, device="cuda")[:0], n_q, n_kv, hd, 1e-6,
                       adjacent_pairs=bool(style), rot_dim=rot, v=dev(v) if store else None, k_cache=kc, v_cache=vc)
    assert be.stats()[1] == d0 + 1  # one launch
    gq, gk = host(tq), host(tk)
    for got, want in ((gq, wq), (gk, wk)):
        if f16:
            assert f16_ulp_diff(got, want) <= TOL_F16_ULP
        else:
            assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want)
    if store:
        rows_used = np.unique(positions)
        assert len(rows_used) == rows or rows > 1  # (duplicates are possible; the later row wins on both sides below)
        wkc, wvc = np.zeros((cap, n_kv * hd), np.uint16), np.zeros((cap, n_kv * hd), np.uint16)
        ora.kv_store_rows(gk, v, positions, wkc, wvc)  # exactly the narrowing of the k this launch produced, v bit-exact
        if len(rows_used) == rows:
            assert np.array_equal(host(kc)[rows_used], wkc[rows_used]) and np.array_equal(host(vc)[rows_used], wvc[rows_used])
        untouched = np.ones(cap, bool)
        untouched[rows_used] = False
        assert not host(kc)[untouched].any() and not host(vc)[untouched].any()
    # the table form on the device: the same angles (apk_rope_table), then the op
    if rot:
        table = be.rope_table(dev(positions), dev(inv))
        assert np.array_equal(host(table).view(np.uint32).reshape(rows, -1), np.asarray(ropes).view(np.uint32).reshape(rows, -1)) or \
            np.max(np.abs(host(table).reshape(rows, -1) - np.asarray(ropes).reshape(rows, -1))) <= 6e-8
        uq, uk = dev(q), dev(k)
        be.qknorm_rope_neox(uq, uk, dev(qw), dev(kw), table, n_q, n_kv, hd, 1e-6, rot_dim=rot) if not style else \
            be.qknorm_rope_norm(uq, uk, dev(qw), dev(kw), table, n_q, n_kv, hd, 1e-6, rot_dim=rot)
        if f16:
            assert f16_ulp_diff(gq, host(uq)) <= 1 and f16_ulp_diff(gk, host(uk)) <= 1
            assert np.mean(gq == host(uq)) > 0.9999
        else:
            assert rel_err_f32(gq, host(uq)) <= 2e-7 and rel_err_f32(gk, host(uk)) <= 2e-7
    # more than a decode-sized batch is declined, nothing launched
    if rows == 64:
        big = torch.zeros((65, n_q * hd), dtype=tq.dtype, device="cuda")
        bigk = torch.zeros((65, n_kv * hd), dtype=tq.dtype, device="cuda")
        with pytest.raises(apk.Declined):
            be.qknorm_rope_pos(big, bigk, dev(qw), dev(kw), torch.zeros(65, dtype=torch.int32, device="cuda"), dev(inv), n_q, n_kv, hd, 1e-6,
                               adjacent_pairs=bool(style), rot_dim=rot)


def test_qknorm_rope_pos_past_capacity_is_flagged_not_faulted(be, ora):
    rows, n_q, n_kv, hd = 3, 2, 1, 128
    q, k, qw, kw, inv, _ = _qk_case(ora, 3, rows, n_q, n_kv, hd, False, [1, 2, 3])
    kc = torch.zeros((4, n_kv * hd), dtype=torch.float16, device="cuda")
    vc = torch.zeros_like(kc)
    with pytest.raises(AssertionError, match="position past capacity"):
        be.qknorm_rope_pos(dev(q), dev(k), dev(qw), dev(kw), dev(np.array([1, 4, 3], np.uint32)), dev(inv), n_q, n_kv, hd, 1e-6,
                           v=dev(k), k_cache=kc, v_cache=vc)
    assert host(kc)[1].any() and host(kc)[3].any() and not host(kc)[[0, 2]].any()


def test_kv_store_position_past_capacity_is_flagged_not_faulted(be, ora):
    rows, n_q, n_kv, hd = 3, 2, 1, 128
    q, k, qw, kw, inv, ropes = _qk_case(ora, 3, rows, n_q, n_kv, hd, False, [1, 2, 3])
    kc = torch.zeros((4, n_kv * hd), dtype=torch.float16, device="cuda")
    vc = torch.zeros_like(kc)
    with pytest.raises(AssertionError, match="position past capacity"):
        be.qknorm_rope_kv_store(dev(q), dev(k), dev(k), dev(qw), dev(kw), dev(ropes), dev(np.array([1, 4, 3], np.uint32)), kc, vc,
                                n_q, n_kv, hd, 1e-6)
    assert host(kc)[1].any() and host(kc)[3].any() and not host(kc)[[0, 2]].any()


# ------------------------------------------------ f32 <-> fp16 activation conversion
def test_cast_is_the_reference_conversion_for_every_pattern(be, ora):
    """allpaka_dtype::f16_to_f32 over all 65 536 half patterns (NaN payloads kept, signalling NaNs not quieted), and
    f32_to_f16 (lib.rs:151-184) over every half value's f32 image, its f32 neighbours, every midpoint between
    consecutive halves (the ties) and their neighbours, the overflow threshold, f32 subnormals, infinities, NaNs of
    every kind, and two million random bit patterns -- bit for bit."""
    halves = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    wide = host(be.cast(dev(halves), torch.float32)).view(np.uint32)
    assert np.array_equal(wide, ora.f16_bits_to_f32(halves).view(np.uint32))
    finite = halves[(halves & 0x7c00) != 0x7c00]
    img = ora.f16_bits_to_f32(finite).view(np.uint32).astype(np.int64)
    nxt = ora.f16_bits_to_f32(((finite & 0x7fff) + 1).astype(np.uint16) | (finite & 0x8000)).view(np.uint32).astype(np.int64)
    mid = (img + nxt) // 2  # adjacent normal halves of one sign: the f32 halfway between them
    sub = (np.arange(0, 2049, dtype=np.float64) * 2.0 ** -25).astype(np.float32)  # halfway between adjacent subnormal halves
    sub = np.concatenate([sub, -sub]).view(np.uint32).astype(np.int64)
    cases = [img + d for d in (-1, 0, 1)] + [mid + d for d in (-1, 0, 1)] + [sub + d for d in (-1, 0, 1)]
    g = np.random.default_rng(77)
    special = np.array([0x7f800000, 0xff800000, 0x7fc00000, 0xffc00000, 0x7f800001, 0xff800001, 0x7fffffff, 0x7fa00000, 0x00000001,
                        0x80000001, 0x007fffff, 0x00800000, 0x33000000, 0x33000001, 0x32ffffff, 0x477fe000, 0x477fefff, 0x477ff000,
                        0x477ff001, 0x7f7fffff, 0xff7fffff, 0, 0x80000000], dtype=np.int64)
    bits = np.concatenate(cases + [special, g.integers(0, 2 ** 32, size=2_000_003, dtype=np.int64)])
    bits = np.clip(bits, 0, 2 ** 32 - 1).astype(np.uint32)
    x = bits.view(np.float32)
    got = host(be.cast(torch.from_numpy(x.copy()).cuda(), torch.float16))
    assert np.array_equal(got, ora.f32_to_f16_bits(x))
    # a length that is not whole tiles, and the declines
    odd = x[:1003].copy()
    assert np.array_equal(host(be.cast(torch.from_numpy(odd).cuda(), torch.float16)), ora.f32_to_f16_bits(odd))
    import allpaka_amd as apk

    t = torch.zeros(16, device="cuda")
    with pytest.raises(apk.Declined):
        apk.lib.check(be.L.apk_cast(be.h, t.data_ptr(), 0, t.data_ptr(), 0, 16))


# ------------------------------------- projection biases, and the whole q/k/v step as one call
@pytest.mark.parametrize("rows,n", [(1, 1024), (6, 5120), (300, 4096), (5, 1001), (64, 24), (3, 7)])
@pytest.mark.parametrize("f16", [False, True])
def test_add_bias_rows(be, ora, rows, n, f16):
    """add_bias_rows (loader.rs:519-523): f32 bit-exact; fp16 rows widened, biased in f32 and rounded once."""
    s = synth()
    g = s.rng(3, rows * 31 + n)
    x, b = s.normal_f32(g, (rows, n)), s.normal_f32(g, n, 0.0, 0.5)
    want = x.copy()
    if f16:
        xb = s.to_f16_bits(x)
        want = ora.f16_bits_to_f32(xb)
        ora.add_bias_rows(want, b)
        want = ora.f32_to_f16_bits(want)
        x = xb
    else:
        ora.add_bias_rows(want, b)
    t = dev(x)
    be.add_bias_rows(t, dev(b))
    assert np.array_equal(host(t), want)


@pytest.mark.parametrize("rows,n_q,n_kv,hd,rot,style", [
    (1, 28, 4, 128, 128, 0),    # Qwen2.5-7B decode: biases, no QK-norm, NeoX
    (6, 28, 4, 128, 128, 0), (300, 40, 8, 128, 128, 0), (2048, 12, 2, 128, 128, 0),
    (33, 32, 2, 128, 64, 0),    # GLM style: biases and partial rotary
    (40, 32, 2, 128, 64, 1), (9, 8, 2, 256, 256, 1), (65, 12, 2, 64, 64, 0), (5, 3, 0, 128, 128, 0), (5, 0, 3, 64, 64, 1),
    (7, 5, 1, 80, 32, 0), (4, 3, 3, 96, 96, 1), (3, 2, 1, 128, 0, 0),   # the element-wise kernel
])
@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("normed", [False, True])
@pytest.mark.parametrize("store", [False, True])
def test_attn_prologue_rows(be, ora, rows, n_q, n_kv, hd, rot, style, f16, normed, store):
    """attention.rs:125-165 + kv.rs:682-697 as one call: add_bias_rows on q, k, v; per-head norm (optional) and the
    row's rotation; k and v narrowed into the cache rows -- against the oracle's ops in the reference's order."""
    import allpaka_amd as apk

    s = synth()
    g = s.rng(3, rows * 577 + n_q * 5 + hd + rot + style)
    q, k, v = s.normal_f32(g, (rows, n_q * hd)), s.normal_f32(g, (rows, n_kv * hd)), s.normal_f32(g, (rows, n_kv * hd))
    qb, kb, vb = s.normal_f32(g, n_q * hd, 0.0, 0.5), s.normal_f32(g, n_kv * hd, 0.0, 0.5), s.normal_f32(g, n_kv * hd, 0.0, 0.5)
    qw, kw = (s.normal_f32(g, hd, 1.0, 0.05), s.normal_f32(g, hd, 1.0, 0.05)) if normed else (None, None)
    if f16:
        q, k, v = s.to_f16_bits(q), s.to_f16_bits(k), s.to_f16_bits(v)
    cap = max(rows + 9, 40)
    positions = g.permutation(cap)[:rows].astype(np.uint32)
    ropes = ora.rope_table([int(p) for p in positions], ora.rope_inv_freq(rot, 1e6)) if rot else np.zeros((rows, 0, 2), np.float32)
    # the oracle, in the reference's order
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6, style=style, q_bias=qb if n_q else None, k_bias=kb if n_kv else None)
    wv = ora.f16_bits_to_f32(v) if f16 else v.copy()
    if n_kv:
        ora.add_bias_rows(wv, vb)
    if f16:
        wv = ora.f32_to_f16_bits(wv)
    wkc, wvc = np.zeros((cap, n_kv * hd), np.uint16), np.zeros((cap, n_kv * hd), np.uint16)
    ora.kv_store_rows(wk, wv, positions, wkc, wvc)
    tq, tk, tv = dev(q), dev(k), dev(v)
    kc = torch.zeros((cap, n_kv * hd), dtype=torch.float16, device="cuda")
    vc = torch.zeros_like(kc)
    rt = dev(ropes) if rot else torch.zeros((rows, 0, 2), device="cuda")
    kw_args = dict(q_bias=dev(qb) if n_q else None, k_bias=dev(kb) if n_kv else None, v_bias=dev(vb) if n_kv else None,
                   q_norm=None if qw is None else dev(qw), k_norm=None if kw is None else dev(kw), adjacent_pairs=bool(style), rot_dim=rot)
    if store:
        kw_args.update(cache_pos=dev(positions), k_cache=kc, v_cache=vc)
    es = 2 if f16 else 4
    tiled = hd in (64, 128, 256) and rot > 0 and (rot % (16 // es) == 0 if style else (rot // 2) % (16 // es) == 0)
    if store and (not tiled or n_kv == 0):  # the cache store rides on the tiled kernels' k items only
        with pytest.raises(apk.Declined):
            be.attn_prologue_rows(tq, tk, tv, n_q, n_kv, hd, 1e-6, rt, **kw_args)
        assert np.array_equal(host(tv), v) and np.array_equal(host(tq), q)  # declined before anything ran
        return
    be.attn_prologue_rows(tq, tk, tv, n_q, n_kv, hd, 1e-6, rt, **kw_args)
    gk = host(tk)
    for got, want in ((host(tq), wq), (gk, wk)):
        if f16:
            assert f16_ulp_diff(got, want) <= TOL_F16_ULP
            assert got.size == 0 or np.mean(got == want) > 0.99  # one rounding of the same f32 chain: equal nearly everywhere
        elif not normed:
            assert np.array_equal(got, want)  # bias and rotation only: the same f32 operations
        else:
            assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want)
    assert np.array_equal(host(tv), wv)  # v + v_bias: one f32 add, rounded once
    if store:
        assert np.array_equal(host(vc), wvc)
        mine_k, mine_v = np.zeros_like(wkc), np.zeros_like(wvc)
        ora.kv_store_rows(gk, wv, positions, mine_k, mine_v)
        assert np.array_equal(host(kc), mine_k)
        assert f16_ulp_diff(host(kc), wkc) <= (TOL_F16_ULP if f16 else 1)


def test_attn_prologue_rows_without_biases_is_the_plain_op(be, ora):
    """No biases: the same kernels as apk_qknorm_rope_kv_store / _neox (two passes per q wave in fp16 included)."""
    rows, n_q, n_kv, hd = 600, 64, 8, 128
    positions = [int(p) for p in np.arange(rows)]
    q, k, qw, kw, inv, ropes = _qk_case(ora, 3, rows, n_q, n_kv, hd, True, positions)
    t1q, t1k, t2q, t2k = dev(q), dev(k), dev(q), dev(k)
    be.qknorm_rope_neox(t1q, t1k, dev(qw), dev(kw), dev(ropes), n_q, n_kv, hd, 1e-6)
    be.attn_prologue_rows(t2q, t2k, None, n_q, n_kv, hd, 1e-6, dev(ropes), q_norm=dev(qw), k_norm=dev(kw))
    assert np.array_equal(host(t1q), host(t2q)) and np.array_equal(host(t1k), host(t2k))


# ------------------------------------------- single-launch layer prologue
@pytest.mark.parametrize("rows,n,n_q,n_kv,hd,f16", [
    (64, 5120, 64, 8, 128, True), (1, 5120, 64, 8, 128, True), (6, 5120, 64, 8, 128, True),
    (1, 1024, 16, 8, 128, False), (8, 2048, 4, 4, 64, False), (3, 1024, 2, 1, 256, True),
    (300, 5120, 64, 8, 128, True),  # beyond the single-launch shape: runs as two launches, same result
])
def test_layer_prologue_matches_the_two_ops(be, ora, rows, n, n_q, n_kv, hd, f16):
    """Continuous-batching decode: every row has its own position; residual add + RMSNorm and
    QK-norm + RoPE go out as one launch and must equal the two reference ops."""
    s = synth()
    g = s.rng(3, rows * 7 + n)
    positions = [int(p) for p in g.integers(0, 32768, size=rows)]
    q, k, qw, kw, inv, ropes = _qk_case(ora, 3, rows, n_q, n_kv, hd, f16, positions)
    x, d = s.normal_f32(g, (rows, n)), s.normal_f32(g, (rows, n))
    gamma = s.normal_f32(g, n, 1.0, 0.05)
    if f16:
        x, d = s.to_f16_bits(x), s.to_f16_bits(d)
    wx, wh, wq, wk = x.copy(), np.zeros_like(x), q.copy(), k.copy()
    ora.add_rmsnorm_rows(wx, d, wh, gamma, 1e-6)
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6)
    tx, th, tq, tk = dev(x), torch.zeros_like(dev(x)), dev(q), dev(k)
    _, d0, _, _ = be.stats()
    be.layer_prologue(tx, dev(d), th, dev(gamma), tq, tk, dev(qw), dev(kw), dev(ropes), n_q, n_kv, hd, 1e-6)
    _, d1, _, _ = be.stats()
    assert d1 - d0 == (1 if rows <= 64 else 2)  # one dispatch for decode batches
    assert np.array_equal(host(tx), wx)
    for got, want in ((host(th), wh), (host(tq), wq), (host(tk), wk)):
        if f16:
            assert f16_ulp_diff(got, want) <= TOL_F16_ULP
        else:
            assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want)


# --------------------------------------------------------------------- SwiGLU
@pytest.mark.parametrize("n", [3072, 512 * 3072, 6 * 25600, 64 * 25600, 1, 5, 1031, 8192 * 768 // 16])
@pytest.mark.parametrize("f16", [False, True])
def test_swiglu(be, ora, n, f16):
    s = synth()
    g = s.rng(4, n)
    gate, up = s.normal_f32(g, n), s.normal_f32(g, n)
    gate[: min(n, 8)] = np.float32([0.0, 1.0, -20.0, 20.0, -88.0, 88.0, -0.0, 1e-30])[: min(n, 8)]
    if f16:
        gate, up = s.to_f16_bits(gate), s.to_f16_bits(up)
    want = gate.copy()
    ora.swiglu(want, up)
    tg = dev(gate)
    be.swiglu(tg, dev(up))
    got = host(tg)
    if f16:
        assert f16_ulp_diff(got, want) <= TOL_F16_ULP
    else:
        assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want)


def test_swiglu_f32_strict_relative_error_over_the_whole_range(be, ora):
    """Element by element (no floor): every normal result within 1e-5 of the reference's
    g / (1 + exp(-g)) * u, from the underflow edge of exp to its overflow edge, and the same
    zeros / infinities / NaNs outside it."""
    g = np.concatenate([np.linspace(-104.0, 104.0, 400001), synth().normal_f32(synth().rng(4, 1), 300000, 0.0, 4.0),
                        [0.0, -0.0, 1e-30, -1e-30, 88.7, -88.7, 88.73, -88.73, -87.3, 120.0, -120.0, 3e38, -3e38, np.inf, -np.inf,
                         np.nan, 0.0]]).astype(np.float32)
    up = np.ones_like(g)
    up[-1] = np.nan
    want = g.copy()
    with np.errstate(all="ignore"):
        ora.swiglu(want, up)
    tg = dev(g)
    be.swiglu(tg, dev(up))
    got = host(tg)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    normal = ok & (np.abs(want) >= np.float32(1.17549435e-38)) & np.isfinite(want)
    rel = np.abs(got[normal].astype(np.float64) - want[normal]) / np.abs(want[normal].astype(np.float64))
    assert rel.max() <= TOL_F32, (rel.max(), g[normal][rel.argmax()])
    rest = ok & ~normal  # zeros, subnormal results, infinities: equal up to one subnormal step
    assert np.all(np.isinf(got[rest]) == np.isinf(want[rest]))
    fin = rest & np.isfinite(want)
    assert np.max(np.abs(got[fin].astype(np.float64) - want[fin])) <= 2e-38
    assert np.array_equal(np.signbit(got[fin & (want == 0)]), np.signbit(want[fin & (want == 0)]))


def test_swiglu_reference_sweep_and_assert(be, ora):
    # ops/mod.rs:172-185
    gate = np.float32([i * 0.7 for i in range(-25, 26)])
    up = np.float32([i * 0.5 - 3.0 for i in range(51)])
    tg = dev(gate)
    be.swiglu(tg, dev(up))
    for got, gg, u in zip(host(tg), gate, up):
        want = ora.silu(gg) * u
        assert abs(got - want) < 1e-5 * (1 + abs(want))
    with pytest.raises(AssertionError):
        be.swiglu(torch.zeros(4, device="cuda"), torch.zeros(3, device="cuda"))


# --------------------------------------------------------------------- GeGLU (tanh)
@pytest.mark.parametrize("n", [2304 * 4, 512 * 9216, 64 * 9216, 1, 5, 1031])
@pytest.mark.parametrize("f16", [False, True])
def test_geglu_tanh(be, ora, n, f16):
    """ops::geglu_tanh (activation.rs:44-51), the FFN gate of the Gemma family.  The device computes
    g * sigmoid(2z) * u, the same function as the reference's 0.5 g (1 + tanh z) u without the cancellation of
    1 + tanh z: to 1e-5 relative where the reference's own rounding of tanh cannot show (1 + tanh z >= 0.1, i.e.
    gates above about -0.9) and to the reference's tolerance idiom |a - b| < 1e-5 (1 + |b|) everywhere."""
    s = synth()
    g = s.rng(4, n + 77)
    gate, up = s.normal_f32(g, n, 0.0, 2.0), s.normal_f32(g, n)
    gate[: min(n, 8)] = np.float32([0.0, 1.0, -20.0, 20.0, -6.0, 6.0, -0.0, 1e-30])[: min(n, 8)]
    if f16:
        gate, up = s.to_f16_bits(gate), s.to_f16_bits(up)
    want = gate.copy()
    ora.geglu_tanh(want, up)
    tg = dev(gate)
    be.geglu_tanh(tg, dev(up))
    got = host(tg)
    if f16:
        # where the reference's rounding of tanh cannot show: 2 ulp; further left its own f32 result is off by
        # parts in 1e3 and more before it is rounded to fp16, so there the reference's tolerance idiom on the values
        gv = gate.view(np.float16).astype(np.float32)
        right = gv >= -0.9
        assert not right.any() or f16_ulp_diff(got[right], want[right]) <= TOL_F16_ULP
        key = lambda b: np.where(b.astype(np.int32) & 0x8000, 0x8000 - b.astype(np.int32), b.astype(np.int32))  # noqa: E731
        a, b = got.view(np.float16).astype(np.float64), want.view(np.float16).astype(np.float64)
        assert np.all((np.abs(key(got) - key(want)) <= TOL_F16_ULP) | (np.abs(a - b) < 1e-5 * (1.0 + np.abs(b))))
    else:
        assert close_idiom(got, want)
        right = gate >= -0.9
        assert not right.any() or rel_err_f32(got[right], want[right]) <= TOL_F32
        # and against the closed form in float64, over the whole range, the device keeps the bar
        gd, ud = gate.astype(np.float64), up.astype(np.float64)
        with np.errstate(over="ignore"):  # 0.5 (1 + tanh z) = 1 / (1 + exp(-2z)), the form that does not cancel in float64 either
            exact = gd * ud / (1.0 + np.exp(-2.0 * np.float64(np.float32(0.7978846)) * gd * (1.0 + np.float64(np.float32(0.044715)) * gd * gd)))
        big = np.abs(exact) > 1e-30
        assert not big.any() or np.max(np.abs(got[big] - exact[big]) / np.abs(exact[big])) <= TOL_F32  # z itself is an f32 product: |2z| ulps in exp(-2z)


def test_geglu_tanh_asserts_equal_lengths(be):
    with pytest.raises(AssertionError):
        be.geglu_tanh(torch.zeros(4, device="cuda"), torch.zeros(3, device="cuda"))


def test_fp16_special_values_follow_the_oracle(be, ora):
    """fp16 edges: sums that overflow to infinity, subnormal inputs and outputs, all-zero rows, signed zeros."""
    n = 1024
    f = lambda a: np.asarray(a, np.float32).astype(np.float16).view(np.uint16)
    x = np.zeros((6, n), np.float32)
    d = np.zeros((6, n), np.float32)
    x[0, :], d[0, :] = 60000.0, 60000.0                    # x + delta = inf in fp16
    x[1, :] = 6e-8 * (1 + np.arange(n) % 7)                # subnormal inputs (fp16 min subnormal 5.96e-8)
    d[1, :] = 6e-8
    x[2, :] = 0.0                                          # zeros + eps: finite, exactly zero
    x[3, ::2], x[3, 1::2] = -0.0, 0.0
    d[3, :] = -0.0
    x[4, :] = np.linspace(-6e-5, 6e-5, n)                  # around the normal/subnormal boundary (6.1e-5)
    x[5, :] = np.linspace(-65504, 65504, n)
    d[5, :] = 0.0
    xb, db = f(x), f(d)
    gamma = np.ones(n, np.float32)
    wx, wh = xb.copy(), np.zeros_like(xb)
    with np.errstate(all="ignore"):
        ora.add_rmsnorm_rows(wx, db, wh, gamma, 1e-6)
    tx, th = dev(xb), torch.zeros_like(dev(xb))
    be.add_rmsnorm_rows(tx, dev(db), th, dev(gamma), 1e-6)
    assert np.array_equal(host(tx), wx)                    # residual sum incl. inf, subnormals and signed zeros
    assert np.all(wx[0] == 0x7C00)
    got = host(th)
    fin = np.isfinite(wh.view(np.float16)) & np.isfinite(got.view(np.float16))
    assert np.array_equal(np.isfinite(wh.view(np.float16)), np.isfinite(got.view(np.float16)))
    assert f16_ulp_diff(got[fin], wh[fin]) <= TOL_F16_ULP
    assert np.all(got[2] == 0)
    # SwiGLU over every finite fp16 gate value, up = 1 and up = -2.5
    gate = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    gate = gate[np.isfinite(gate.view(np.float16))]
    for upv in (1.0, -2.5):
        up = f(np.full(gate.size, upv))
        want = gate.copy()
        with np.errstate(all="ignore"):
            ora.swiglu(want, up)
        tg = dev(gate)
        be.swiglu(tg, dev(up))
        g_ = host(tg)
        assert np.array_equal(np.isfinite(g_.view(np.float16)), np.isfinite(want.view(np.float16)))
        ok = np.isfinite(want.view(np.float16))
        assert f16_ulp_diff(g_[ok], want[ok]) <= TOL_F16_ULP, upv


# ------------------------------------------------- residual add, softmax alone
@pytest.mark.parametrize("n", [1, 3, 8, 1024, 5120 * 6 + 5, 65536 * 3 + 1])
@pytest.mark.parametrize("f16", [False, True])
def test_add_assign_slice_bit_exact(be, ora, n, f16):
    s = synth()
    g = s.rng(1, n)
    a, b = s.normal_f32(g, n), s.normal_f32(g, n)
    if f16:
        a16, b16 = s.to_f16_bits(a), s.to_f16_bits(b)
        want = ora.f32_to_f16_bits(ora.f16_bits_to_f32(a16) + ora.f16_bits_to_f32(b16))
        ta, tb = dev(a16), dev(b16)
    else:
        want = a.copy()
        ora.add_assign_slice(want, b)
        ta, tb = dev(a), dev(b)
    be.add_assign_slice(ta, tb)
    assert np.array_equal(host(ta), want)
    assert np.array_equal(host(tb), b16 if f16 else b)  # the addend is only read
    with pytest.raises(AssertionError):  # blas.rs: a shorter source panics (ops/mod.rs:394-408)
        be.add_assign_slice(ta, tb[:-1])


@pytest.mark.parametrize("n", [1, 3, 8, 1024, 2048, 5120 * 6 + 5, 65536 * 3 + 1])
@pytest.mark.parametrize("f16", [False, True])
def test_add_scaled_slice_bit_exact(be, ora, n, f16):
    """ops::add_scaled_slice (blas.rs:25-102): dst = fma(src, scale, dst), one rounding -- bit for bit the oracle's fmaf
    (an unfused scale * src + dst differs from it in about a quarter of the elements, so a device multiply-then-add
    would fail here); with fp16 rows the f32 fma rounded once."""
    s = synth()
    g = s.rng(2, n)
    a, b = s.normal_f32(g, n), s.normal_f32(g, n)
    for scale in (0.37109375, 1.0, -2.5e-3):
        if f16:
            a16, b16 = s.to_f16_bits(a), s.to_f16_bits(b)
            w32 = ora.f16_bits_to_f32(a16)
            ora.add_scaled_slice(w32, ora.f16_bits_to_f32(b16), scale)
            want = ora.f32_to_f16_bits(w32)
            ta, tb = dev(a16), dev(b16)
        else:
            want = a.copy()
            ora.add_scaled_slice(want, b, scale)
            if n >= 1024 and scale == 0.37109375:  # the check has teeth: the unfused form is a different result
                assert np.mean((np.float32(scale) * b + a).astype(np.float32) != want) > 0.05
            ta, tb = dev(a), dev(b)
        be.add_scaled_slice(ta, tb, scale)
        assert np.array_equal(host(ta), want)
        assert np.array_equal(host(tb), b16 if f16 else b)  # the source is only read
    with pytest.raises(AssertionError):  # a shorter source panics (ops/mod.rs:403-408)
        be.add_scaled_slice(ta, tb[:-1], 2.0)
    import allpaka_amd as apk

    with pytest.raises(apk.Declined):  # dst and src are two tensors (a unique borrow and a shared one in the reference)
        be.add_scaled_slice(ta, ta, 2.0)


def test_decode_moe_combine_is_add_scaled_slice_per_pick(be, ora):
    """The single-token combine (moe.rs:500-509): out = 0, then add_scaled_slice(out, down_i, weight_i) per picked
    expert, best first, then the shared expert with weight 1.  Three ways here, one result: that loop on the oracle,
    the same loop through apk_add_scaled, and apk_moe_combine_add_rmsnorm with no tok_off (hits listed in pick order)
    on a zero residual."""
    s = synth()
    hidden, k = 2048, 8
    g = s.rng(3, hidden)
    downs = s.normal_f32(g, (k + 1, hidden))
    logits = s.normal_f32(g, 128)
    _ids, w = ora.route_gated(logits, k)  # best first
    weights = [float(v) for v in w] + [1.0]
    want = np.zeros(hidden, np.float32)
    for i in range(k + 1):
        ora.add_scaled_slice(want, downs[i], weights[i])
    out = dev(np.zeros(hidden, np.float32))
    td = dev(downs)
    for i in range(k + 1):
        be.add_scaled_slice(out, td[i], weights[i])
    assert np.array_equal(host(out), want)
    x = dev(np.zeros((1, hidden), np.float32))
    hit_row = dev(np.arange(k + 1, dtype=np.uint32))
    hit_w = dev(np.asarray(weights, np.float32))
    be.moe_combine_add_rmsnorm(x, td, None, hit_row, hit_w, None, None, 1e-6)
    assert np.array_equal(host(x)[0], want)


@pytest.mark.parametrize("rows,n", [(1, 3), (1, 128), (5, 256), (1024, 128), (3, 1000), (2, 4096)])
def test_softmax_rows(be, ora, rows, n):
    s = synth()
    x = s.normal_f32(s.rng(4, rows * 7 + n), (rows, n), 0.0, 3.0)
    want = x.copy()
    for r in range(rows):
        ora.softmax(want[r])
    t = dev(x)
    be.softmax(t)
    got = host(t)
    assert rel_err_f32(got, want) <= TOL_F32
    assert np.allclose(got.sum(axis=1, dtype=np.float64), 1.0, atol=1e-5)
    # the reference's vectors (ops/mod.rs:147-161): order kept, sums to 1; huge logits stay finite
    v = dev(np.float32([1.0, 3.0, 2.0]))
    be.softmax(v)
    h = host(v)
    assert h[1] > h[2] > h[0] and abs(h.sum() - 1.0) < 1e-6
    v = dev(np.float32([1000.0, 999.0]))
    be.softmax(v)
    assert np.all(np.isfinite(host(v))) and abs(host(v).sum() - 1.0) < 1e-6
    import allpaka_amd as apk

    with pytest.raises(apk.Declined):  # vocabulary-sized rows: the sequential f32 sum is not reproducible to 1e-5
        be.softmax(torch.zeros(4097, device="cuda"))


# --------------------------------------------------------------------- router
def _ref_logits(n):
    return np.float32([((i * 37 % 331) - 165.0) * 0.03 for i in range(n)])


@pytest.mark.parametrize("rows,n_expert,k", [(1024, 128, 8), (1, 128, 8), (7, 64, 4), (33, 256, 8), (5, 60, 6), (3, 4, 4), (9, 200, 1),
                                            (40, 257, 8), (17, 384, 6), (5, 1024, 8), (3, 1000, 64), (33, 65, 8), (12, 100, 64), (6, 129, 8),
                                            (9, 64, 64)])
@pytest.mark.parametrize("norm,scale", [(True, 1.0), (False, 1.5)])
def test_route_topk(be, ora, rows, n_expert, k, norm, scale):
    s = synth()
    logits = s.normal_f32(s.rng(4, rows * n_expert + k), (rows, n_expert))
    want_ids, want_w = ora.route_rows(logits, k, ora.SOFTMAX, norm, scale, threads=4)
    ids, w = be.route_rows(dev(logits), k, norm=norm, scale=scale)
    assert np.array_equal(host(ids), want_ids)  # bit-exact indices
    # the device's scores are the reference's bit for bit (its libm's expf, its one-after-the-other sum), so the weights are too
    assert np.array_equal(host(w).view(np.uint32), want_w.view(np.uint32))


def test_route_where_distinct_logits_share_a_score(be, ora):
    """The reference selects on the scores (moe.rs:552-582), so two DISTINCT logits that round to one score are a tie
    there, broken by the lower index -- where an order taken on the raw logits puts the larger logit first.  Rows built
    by search on the CPU: a pair inside the top-k, a pair straddling its boundary, scores that underflow to zero next to
    masked (-inf) experts, and sigmoid scores that saturate at 1.  On each the two orders differ (asserted, or the row
    pins nothing) and the device takes the reference's."""
    import allpaka_amd as apk

    s = synth()
    g = s.rng(4, 4242)

    def pair_with_one_score(row, i, j, lo, hi, k):
        """row[i] = v, row[j] = the next float above v, for the first v in [lo, hi) where the oracle's scores are equal"""
        v = np.float32(lo)
        while v < hi:
            row[i], row[j] = v, np.nextafter(v, np.float32(np.inf))
            sc = row.copy()
            ora.softmax(sc)
            if sc[i] == sc[j] and row[i] != row[j]:
                return
            v = np.nextafter(np.float32(v + 1e-3), np.float32(np.inf))
        raise AssertionError("no collapsing pair found")

    rows = []
    a = (0.3 * s.normal_f32(g, 128) - 3.0).astype(np.float32)  # everything else well below
    a[5] = 8.0  # the pair's spacing (an ulp of 0.1) is far below an ulp of logit - max
    pair_with_one_score(a, 10, 20, 0.05, 0.5, 8)  # both inside the top 8: the reference lists 10 before 20
    rows.append((a, 8, ora.SOFTMAX))
    b = (0.3 * s.normal_f32(g, 128) - 3.0).astype(np.float32)
    b[[1, 2, 3, 4, 6, 7, 8]] = np.float32([9.0, 8.5, 8.0, 7.9, 7.8, 7.7, 7.6])  # seven sure picks
    pair_with_one_score(b, 30, 40, 0.05, 0.5, 8)  # the eighth: index 30 by the scores, index 40 by the logits
    rows.append((b, 8, ora.SOFTMAX))
    c = s.normal_f32(g, 128)
    c[0] = 200.0  # every other score underflows to zero: the rest of the picks are the lowest indices
    c[[2, 3]] = -np.inf
    rows.append((c, 8, ora.SOFTMAX))
    d = s.normal_f32(g, 64)
    d[[50, 9, 33]] = np.float32([21.0, 20.0, 30.0])  # sigmoid saturates at 1.0f for all three
    rows.append((d, 4, ora.SIGMOID))
    for row, k, gating in rows:
        want_ids, want_w = ora.route_gated(row, k, gating, True, 1.0)
        if gating == ora.SOFTMAX:
            assert not np.array_equal(want_ids, ora.topk_by_logits(row, k)), "the row does not separate the two orders"
        got = be.route_gated(dev(row), k, apk.Gating.Softmax if gating == ora.SOFTMAX else apk.Gating.Sigmoid, True, 1.0)
        assert [e for e, _ in got] == list(want_ids), (list(want_ids), got)
        assert np.array_equal(np.float32([x for _, x in got]), want_w)
    assert list(ora.route_gated(rows[0][0], 8)[0]).index(10) + 1 == list(ora.route_gated(rows[0][0], 8)[0]).index(20)
    assert 30 in ora.route_gated(rows[1][0], 8)[0] and 40 not in ora.route_gated(rows[1][0], 8)[0]
    assert list(ora.route_gated(rows[2][0], 8)[0]) == [0, 1, 2, 3, 4, 5, 6, 7]
    assert list(ora.route_gated(rows[3][0], 4, ora.SIGMOID)[0])[:3] == [9, 33, 50]


def test_router_exp_is_the_host_libm_exp_over_its_whole_range(be, ora):
    """The device restates glibc's expf; sigmoid gating without renormalisation returns 1 / (1 + expf(-logit)) for
    every expert (k = n), so a sweep of logits from below the underflow edge to above the overflow edge compares the two
    implementations bit for bit: 2 M arguments, every binade of the range, the special values and the branch edges."""
    import allpaka_amd as apk

    g = synth().rng(4, 99)
    n, rows = 64, 32768
    mag = np.exp(g.uniform(np.log(1e-8), np.log(120.0), size=rows * n)).astype(np.float32)
    x = (mag * np.where(g.integers(0, 2, size=rows * n) == 1, 1, -1)).astype(np.float32)
    edges = np.float32([0.0, -0.0, 88.0, -88.0, 88.72283, 88.72284, 88.7228, -103.97, -103.972, -103.98, -103.27, -103.28, 104.0, -104.0,
                        np.inf, -np.inf, 87.99999, -87.99999, 1e-30, -1e-30, 0.5, -0.5, 17.328, -17.328])
    x[: len(edges)] = edges
    x = x.reshape(rows, n)
    ids, w = be.route_rows(dev(x), n, gating=apk.Gating.Sigmoid, norm=False, scale=1.0)
    want_ids, want_w = ora.route_rows(x, n, ora.SIGMOID, False, 1.0, threads=4)
    assert np.array_equal(host(ids), want_ids)
    assert np.array_equal(host(w).view(np.uint32), want_w.view(np.uint32))
    # softmax rows spread over the same range (arguments logit - max from 0 down to -220)
    y = (-np.abs(x[:2048]) * 1.9).astype(np.float32)
    y[:, 0] = 0.0
    ids, w = be.route_rows(dev(y), 8, gating=apk.Gating.Softmax, norm=False, scale=1.0)
    want_ids, want_w = ora.route_rows(y, 8, ora.SOFTMAX, False, 1.0, threads=4)
    assert np.array_equal(host(ids), want_ids) and np.array_equal(host(w).view(np.uint32), want_w.view(np.uint32))


def test_route_on_probabilities_is_the_older_route(be, ora):
    """model::route(probs, k) (moe.rs:623-658): the rows are scores already.  The reference's own vector
    (tests/gpu_eligible_forward.rs:89-97) and random softmaxed rows, ids and weights bit for bit."""
    got = be.route(dev(np.float32([0.1, 0.5, 0.15, 0.25])), 2)
    assert [e for e, _ in got] == [1, 3]
    assert np.array_equal(np.float32([x for _, x in got]), np.float32([0.5, 0.25]) / (np.float32(0.5) + np.float32(0.25)))
    wi, ww = ora.route(np.float32([0.1, 0.5, 0.15, 0.25]), 2)
    assert list(wi) == [1, 3] and np.array_equal(np.float32([x for _, x in got]), ww)
    g = synth().rng(4, 4242)
    for n, k in ((128, 8), (64, 1), (256, 8), (1000, 25), (7, 7), (5, 9)):
        probs = synth().normal_f32(g, n)
        ora.softmax(probs)
        if n == 128:
            probs[17] = probs[90] = probs[3]  # equal scores: lower index first
        wi, ww = ora.route(probs, k)
        got = be.route(dev(probs), k)
        assert [e for e, _ in got] == list(wi) and np.array_equal(np.float32([x for _, x in got]), ww), (n, k)
    zero = be.route(dev(np.zeros(6, np.float32)), 3)  # total == 0: 1 / k each
    assert [e for e, _ in zero] == [0, 1, 2] and all(x == np.float32(1.0) / np.float32(3.0) for _, x in zero)
    assert be.route(dev(np.zeros(4, np.float32))[:0], 3) == []


def test_route_reference_vectors_ties_sigmoid_bias(be, ora):
    import allpaka_amd as apk

    base = _ref_logits(256)  # moe.rs:664-715
    for gating, norm in [(apk.Gating.Softmax, True), (apk.Gating.Softmax, False), (apk.Gating.Sigmoid, True)]:
        for k in (1, 8):
            wi, ww = ora.route_gated(base, k, int(gating), norm, 1.5)
            got = be.route_gated(dev(base), k, gating, norm, 1.5)
            assert [e for e, _ in got] == list(wi)
            assert np.array_equal(np.float32([x for _, x in got]), ww)
    bias = np.float32([0.5 + (i % 7) * 0.01 for i in range(256)])
    wi, ww = ora.route_gated(base, 8, ora.SIGMOID, True, 2.5, bias)
    got = be.route_gated(dev(base), 8, apk.Gating.Sigmoid, True, 2.5, dev(bias))
    assert [e for e, _ in got] == list(wi) and np.array_equal(np.float32([x for _, x in got]), ww)
    # softmax with a selection bias: selection on score + bias, weights from the scores
    lg = synth().normal_f32(synth().rng(4, 5), 128)
    b2 = synth().normal_f32(synth().rng(4, 6), 128, 0.0, 0.01)
    wi, ww = ora.route_gated(lg, 8, ora.SOFTMAX, True, 1.0, b2)
    got = be.route_gated(dev(lg), 8, apk.Gating.Softmax, True, 1.0, dev(b2))
    assert [e for e, _ in got] == list(wi) and np.array_equal(np.float32([x for _, x in got]), ww)
    # exact ties: the lower index wins, inside the top-k and at its boundary
    t = np.zeros(128, np.float32)
    t[[3, 9, 12, 100]] = 2.0
    t[[5, 7, 77]] = 1.0
    got = be.route_gated(dev(t), 6)
    assert [e for e, _ in got] == [3, 9, 12, 100, 5, 7] == list(ora.route_gated(t, 6)[0])
    got = be.route_gated(dev(np.zeros(8, np.float32)), 2)
    assert [e for e, _ in got] == [0, 1] and np.allclose([x for _, x in got], 0.5)
    # route(probs, k) of the reference's test (gpu_eligible_forward.rs:88-97) through log-probabilities
    got = be.route_gated(dev(np.log(np.float32([0.1, 0.5, 0.15, 0.25]))), 2)
    assert [e for e, _ in got] == [1, 3] and abs(got[0][1] - 2 / 3) < 1e-6 and abs(got[1][1] - 1 / 3) < 1e-6
    # k clamps to n
    assert len(be.route_gated(dev(t[:4].copy()), 8)) == 4
    # the reference's stack/heap boundary (moe.rs:680-715): a 257th expert that can never win leaves
    # the picks and weights of the 256-expert router as they were, for every gating
    wide = np.append(base, np.float32(-np.inf))
    for gating, norm in [(apk.Gating.Softmax, True), (apk.Gating.Softmax, False), (apk.Gating.Sigmoid, True)]:
        for k in (1, 8):
            a, b = be.route_gated(dev(base), k, gating, norm, 1.5), be.route_gated(dev(wide), k, gating, norm, 1.5)
            assert [e for e, _ in a] == [e for e, _ in b]
            assert np.allclose([x for _, x in a], [x for _, x in b], rtol=0, atol=1e-6)
    wide_bias = np.append(bias, np.float32(0.0))
    a = be.route_gated(dev(base), 8, apk.Gating.Sigmoid, True, 2.5, dev(bias))
    b = be.route_gated(dev(wide), 8, apk.Gating.Sigmoid, True, 2.5, dev(wide_bias))
    assert [e for e, _ in a] == [e for e, _ in b] and np.allclose([x for _, x in a], [x for _, x in b], rtol=0, atol=1e-6)
    # wide routers pick the true top-k, best first (moe.rs:719-726)
    w320 = _ref_logits(320)
    got = be.route_gated(dev(w320), 4, apk.Gating.Softmax, False, 1.0)
    assert [e for e, _ in got] == list(np.argsort(-w320, kind="stable")[:4]) == list(ora.route_gated(w320, 4, ora.SOFTMAX, False, 1.0)[0])
    # more than 1024 experts is declined
    with pytest.raises(apk.Declined):
        be.route_gated(dev(np.zeros(1025, np.float32)), 4)


@pytest.mark.parametrize("rows,n_expert,k", [(1, 128, 8), (6, 128, 8), (16, 128, 8), (16, 64, 6), (13, 256, 8), (16, 1024, 64), (5, 512, 10),
                                            (16, 16, 16), (1, 4, 4), (15, 60, 3), (9, 128, 16), (12, 1000, 25), (2, 64, 64), (16, 65, 1),
                                            # beyond one launch: the two entries run
                                            (17, 128, 8), (64, 128, 8), (300, 24, 5), (1024, 128, 8), (2049, 128, 8)])
@pytest.mark.parametrize("gating", ["softmax", "sigmoid_bias"])
def test_route_group_equals_router_then_grouping(be, ora, rows, n_expert, k, gating):
    """The one-launch router + grouping of a decode-sized batch against the oracle, and bit for bit against
    apk_route_topk followed by apk_moe_permute."""
    import allpaka_amd as apk

    s = synth()
    g = s.rng(4, rows * 131 + n_expert + k)
    logits = s.normal_f32(g, (rows, n_expert))
    if n_expert > 8:
        logits[:, n_expert // 3] = -60.0  # an expert nobody picks (k < n_expert - 1 in these cases)
    bias = s.normal_f32(g, n_expert, 0.0, 0.01) if gating == "sigmoid_bias" else None
    kind = apk.Gating.Sigmoid if bias is not None else apk.Gating.Softmax
    args = dict(gating=kind, norm=True, scale=1.25, bias=None if bias is None else dev(bias))
    (ids, w), got = be.route_group(dev(logits), k, **args)
    ids2, w2 = be.route_rows(dev(logits), k, **args)
    want = be.moe_permute(ids2, w2, n_expert)
    assert torch.equal(ids, ids2) and torch.equal(w, w2)
    for name, a, b in zip(["table", "tok", "tok_off", "hit_row", "hit_w"], got, want):
        assert a.shape == b.shape and torch.equal(a, b), name
    o_ids, o_w = ora.route_rows(logits, k, ora.SIGMOID if bias is not None else ora.SOFTMAX, True, 1.25, bias, threads=4)
    assert np.array_equal(host(ids), o_ids) and rel_err_f32(host(w), o_w) <= TOL_F32
    for name, a, b in zip(["table", "tok", "tok_off", "hit_row"], got, ora.moe_group(o_ids, o_w, n_expert)):
        assert np.array_equal(host(a), b), name
    assert be.take_faults() == 0


# ------------------------------------------------------- grouping and gather
@pytest.mark.parametrize("rows,k,n_expert", [(1024, 8, 128), (1, 8, 128), (5, 2, 4), (600, 8, 16), (64, 1, 256), (777, 3, 7), (2048, 8, 128),
                                             # beyond 2048 tokens: the two-launch form (parts of 1024 tokens)
                                             (2049, 3, 7), (5000, 8, 128), (4096, 8, 256), (3000, 1, 1000), (7001, 6, 60)])
def test_moe_permute_and_gather_bit_exact(be, ora, rows, k, n_expert):
    s = synth()
    g = s.rng(4, rows + k)
    logits = s.normal_f32(g, (rows, n_expert))
    if rows > 4:
        logits[:, n_expert // 2] = -50.0  # an expert nobody picks: the table must skip it
    ids, w = ora.route_rows(logits, k, threads=4)
    want = ora.moe_group(ids, w, n_expert)
    got = be.moe_permute(dev(ids), dev(w), n_expert)
    names = ["table", "tok", "tok_off", "hit_row", "hit_w"]
    for name, a, b in zip(names, got, want):
        a = host(a)
        assert a.shape == b.shape, name
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), name
    for f16 in (False, True):
        cols = 2048 if rows <= 1024 else 256
        hs = s.normal_f32(g, (rows, cols))
        if f16:
            hs = s.to_f16_bits(hs)
        xe = be.gather_rows(dev(hs), got[1])
        assert np.array_equal(host(xe), ora.gather_rows(hs, want[1]))
        xs = be.scatter_rows(dev(hs), got[3], k)  # token-side form of the same permutation
        assert torch.equal(xs, xe)


@pytest.mark.parametrize("rows,k,n_expert,n,f16", [(1024, 8, 128, 2048, False), (1, 8, 128, 2048, False), (33, 4, 16, 512, True),
                                                    (300, 8, 128, 2048, True), (7, 1, 4, 8192, False), (5, 3, 8, 64, True)])
def test_moe_combine_add_rmsnorm(be, ora, rows, k, n_expert, n, f16):
    import allpaka_amd as apk

    s = synth()
    g = s.rng(4, rows * 5 + n)
    logits = s.normal_f32(g, (rows, n_expert))
    ids, w = ora.route_rows(logits, k, threads=4)
    table, tok, tok_off, hit_row, hit_w = ora.moe_group(ids, w, n_expert)
    flat = s.normal_f32(g, (rows * k, n))
    x = s.normal_f32(g, (rows, n))
    gamma = s.normal_f32(g, n, 1.0, 0.05)
    if f16:
        flat, x = s.to_f16_bits(flat), s.to_f16_bits(x)
    wx, wh = x.copy(), np.zeros_like(x)
    ora.moe_combine_add_rmsnorm(wx, flat, tok_off, hit_row, hit_w, wh, gamma, 1e-6)
    tx, th = dev(x), torch.zeros_like(dev(x))
    be.moe_combine_add_rmsnorm(tx, dev(flat), dev(tok_off), dev(hit_row), dev(hit_w), th, dev(gamma), 1e-6)
    assert np.array_equal(host(tx), wx)  # fma per hit in CSR order, then one add: bit-exact
    if f16:
        assert f16_ulp_diff(host(th), wh) <= TOL_F16_ULP
    else:
        assert rel_err_f32(host(th), wh) <= TOL_F32 and close_idiom(host(th), wh)
    tx2 = dev(x)
    be.moe_combine_add_rmsnorm(tx2, dev(flat), dev(tok_off), dev(hit_row), dev(hit_w), None, None, 1e-6)
    assert torch.equal(tx2, tx)
    # without the tok_off list: every token has k hits, at [t*k, (t+1)*k) -- the same launch minus one dependent load
    assert np.array_equal(tok_off, np.arange(rows + 1, dtype=np.uint32) * k)
    tx3, th3 = dev(x), torch.zeros_like(dev(x))
    be.moe_combine_add_rmsnorm(tx3, dev(flat), None, dev(hit_row), dev(hit_w), th3, dev(gamma), 1e-6)
    assert torch.equal(tx3, tx) and torch.equal(th3, th)
    if rows > 1:  # hits that do not divide among the tokens cannot do without the list
        with pytest.raises(apk.Declined):
            be.moe_combine_add_rmsnorm(dev(x), dev(flat)[:-1], None, dev(hit_row), dev(hit_w), None, None, 1e-6)


@pytest.mark.parametrize("rows,k,n_expert,n,f16", [(1024, 8, 128, 2048, False), (1, 8, 128, 2048, True), (33, 4, 16, 512, True),
                                                    (300, 6, 64, 1024, False), (7, 1, 4, 256, False)])
def test_moe_shared_expert_hits(be, ora, rows, k, n_expert, n, f16):
    """GLM-style layers: the shared expert's rows follow the routed experts' rows and every token takes one more hit of
    weight 1 there (prefill.rs:621-635).  Device grouping -> lengthened lists -> combine, against the oracle's."""
    s = synth()
    g = s.rng(4, rows * 11 + n + k)
    logits = s.normal_f32(g, (rows, n_expert))
    ids, w = ora.route_rows(logits, k, threads=4)
    table, tok, tok_off, hit_row, hit_w = ora.moe_group(ids, w, n_expert)
    wto, whr, whw = ora.moe_shared_hits(tok_off, hit_row, hit_w, rows * k)
    got = be.moe_permute(dev(ids), dev(w), n_expert)
    gto, ghr, ghw = be.moe_shared_hits(got[2], got[3], got[4], rows * k)
    assert np.array_equal(host(gto), wto) and np.array_equal(host(ghr), whr) and np.array_equal(host(ghw), whw)
    assert whr.reshape(rows, k + 1)[:, k].tolist() == list(range(rows * k, rows * k + rows)) and (whw.reshape(rows, k + 1)[:, k] == 1).all()
    flat = s.normal_f32(g, (rows * k + rows, n))  # the routed experts' down rows, then the shared expert's
    x = s.normal_f32(g, (rows, n))
    gamma = s.normal_f32(g, n, 1.0, 0.05)
    if f16:
        flat, x = s.to_f16_bits(flat), s.to_f16_bits(x)
    wx, wh = x.copy(), np.zeros_like(x)
    ora.moe_combine_add_rmsnorm(wx, flat, wto, whr, whw, wh, gamma, 1e-6)
    tx, th = dev(x), torch.zeros_like(dev(x))
    be.moe_combine_add_rmsnorm(tx, dev(flat), gto, ghr, ghw, th, dev(gamma), 1e-6)
    assert np.array_equal(host(tx), wx)
    if f16:
        assert f16_ulp_diff(host(th), wh) <= TOL_F16_ULP
    else:
        assert rel_err_f32(host(th), wh) <= TOL_F32 and close_idiom(host(th), wh)
    import allpaka_amd as apk

    with pytest.raises(apk.Declined):  # the lengthened lists need arrays of their own
        apk.lib.check(be.L.apk_moe_shared_hits(be.h, got[2].data_ptr(), got[3].data_ptr(), got[4].data_ptr(), rows, rows * k,
                                               got[2].data_ptr(), ghr.data_ptr(), ghw.data_ptr()))


@pytest.mark.parametrize("rows,n", [(1, 151936), (64, 151936), (3, 1000), (5, 7), (2, 16384), (300, 4096), (2048, 4096), (17, 8196),
                                    (128, 262144), (40, 20000), (16, 151937)])
def test_argmax_rows(be, ora, rows, n):
    """(128, 262144) is the largest grid the host produces (rows * parts = 8192 workgroups, 64 arrivals per row);
    (2048, 4096) and (17, 8196) leave lanes with re-read tiles next to live ones; (16, 151937) is a ragged row."""
    g = synth().rng(5, rows + n)
    logits = synth().normal_f32(g, (rows, n))
    if n >= 1000:
        logits[0, [17, 900, 333]] = 9.0  # exact ties: the higher index wins
        if rows > 1:
            logits[1, :] = -1.5  # all equal: the last index
        if rows > 2:
            logits[2, :] = -np.abs(logits[2, :])  # every value negative: the integer order of the bits is reversed
            logits[2, [5, n - 3]] = -0.0  # the largest of them, twice
        if rows > 4:
            logits[3, [40, n // 2]] = np.float32(np.nan)  # +NaN is the largest value under total_cmp, the last one wins
            logits[4, n // 3] = np.float32(np.inf)
            logits[4, 7] = -np.float32(np.nan)  # -NaN is the smallest
            for r in range(5, rows):  # planted ties at random places, some a workgroup part apart, some in one lane's tiles
                m = np.float32(logits[r].max() + 1.0)
                at = g.integers(0, n, size=3)
                logits[r, at] = m
                logits[r, min(int(at[0]) + 2048, n - 1)] = m
    want = [ora.argmax_last(logits[r]) for r in range(rows)]
    x = dev(logits)
    for _ in range(2):  # the per-row scratch is re-armed by the kernel: a second call sees clean state
        got = host(be.argmax_rows(x))
        assert got.tolist() == want
    if n >= 1000:
        assert want[0] == 900 and (rows == 1 or want[1] == n - 1) and (rows <= 2 or want[2] == n - 3)
        assert rows <= 4 or (want[3] == n // 2 and want[4] == n // 3)


def test_permute_declines_and_faults(be):
    import allpaka_amd as apk

    ids = torch.tensor([[0, 9]], dtype=torch.int32, device="cuda")  # expert 9 of 4
    w = torch.ones((1, 2), device="cuda")
    be.moe_permute(ids, w, 4)
    assert be.take_faults() & 2
    with pytest.raises(apk.Declined):
        be.moe_permute(ids, w, 2000)
    src = torch.ones((2, 64), device="cuda")
    out = be.gather_rows(src, torch.tensor([1, 7], dtype=torch.int32, device="cuda"))
    assert be.take_faults() & 4 and np.all(host(out)[0] == 1.0)
    with pytest.raises(apk.Declined):
        be.gather_rows(torch.ones((2, 3), device="cuda"), torch.tensor([0], dtype=torch.int32, device="cuda"))
    out = be.scatter_rows(src, torch.tensor([1, 9, 0, 3], dtype=torch.int32, device="cuda"), 2)
    assert be.take_faults() & 4 and np.all(host(out)[[0, 1, 3]] == 1.0)


def test_family_step_entries_decline_and_leave_their_tensors_alone(be):
    """NULL arguments, unsupported types, misaligned tensors and impossible geometry are declined (a positive status
    with a message) by the entries of the Gemma / Qwen2 / GLM steps, before anything is launched."""
    import ctypes as C

    import allpaka_amd.lib as lib

    L, h = be.L, be.h
    t = torch.ones(1024, device="cuda")
    before = t.clone()
    ptr = t.data_ptr()

    def declined(rc, code):
        assert rc == code, (rc, L.apk_last_error())
        assert L.apk_last_error()  # a message is left for the caller

    declined(L.apk_cast(h, ptr, 0, ptr + 2048, 7, 16), 1)            # unknown type
    declined(L.apk_cast(h, None, 0, ptr, 1, 16), 3)                  # NULL
    declined(L.apk_cast(h, ptr + 4, 0, ptr + 2048, 1, 16), 2)        # misaligned
    declined(L.apk_add_bias_rows(h, ptr, None, 2, 64, 0), 3)
    declined(L.apk_add_bias_rows(h, ptr, ptr + 2048, 2, 64, 5), 1)
    declined(L.apk_add_bias_rows(h, ptr + 4, ptr + 2048, 2, 64, 0), 2)
    assert L.apk_add_bias_rows(h, None, None, 0, 64, 0) == 0          # no rows: nothing to do
    declined(L.apk_postnorm_add_rmsnorm_rows(h, ptr, ptr, ptr + 2048, ptr + 1024, ptr + 2048, 64, 2, 1e-6, 0), 2)  # x aliases delta
    declined(L.apk_postnorm_add_rmsnorm_rows(h, ptr, ptr + 512, None, ptr + 1024, ptr + 2048, 64, 2, 1e-6, 0), 3)
    declined(L.apk_moe_shared_hits(h, None, ptr, ptr, 2, 4, ptr + 1024, ptr + 2048, ptr + 3072), 3)
    declined(L.apk_attn_prologue_rows(h, None), 3)
    a = lib.AttnPrologue()
    a.q, a.k, a.rope = ptr, ptr + 2048, ptr
    a.rows, a.n_q, a.n_kv, a.head_dim, a.rot_dim, a.eps, a.dtype = 1, 2, 1, 128, 128, 1e-6, 0
    a.q_bias = ptr + 4                                                # misaligned bias
    declined(L.apk_attn_prologue_rows(h, C.byref(a)), 2)
    a.q_bias = None
    a.rot_dim = 130                                                   # wider than the head
    declined(L.apk_attn_prologue_rows(h, C.byref(a)), 2)
    a.rot_dim, a.dtype = 128, 9
    declined(L.apk_attn_prologue_rows(h, C.byref(a)), 1)
    a.dtype, a.k_cache = 0, ptr                                       # a cache store without v / positions
    declined(L.apk_attn_prologue_rows(h, C.byref(a)), 3)
    a.k_cache, a.head_dim, a.rot_dim, a.v_bias = None, 96, 96, ptr    # v_bias without v (and no store)
    declined(L.apk_attn_prologue_rows(h, C.byref(a)), 3)
    be.sync()
    assert torch.equal(t, before)


@pytest.mark.parametrize("rows,k,cols,f16", [(600, 8, 3600, False), (600, 8, 3600, True), (3, 2, 8200, False), (4099, 1, 520, True),
                                             (9, 64, 4, False)])
def test_scatter_rows_is_the_permutation(be, rows, k, cols, f16):
    """dst[hit_row[t*k + j]] = src[t] for any permutation of the rows, bit for bit: both slice widths
    (outputs under and over 64 MiB), rows that end inside a slice, slice counts that do not fill the last
    group of eight workgroups."""
    gen = torch.Generator(device="cuda").manual_seed(rows * 31 + cols)
    src = torch.randn((rows, cols), generator=gen, device="cuda")
    if f16:
        src = src.half()
    hit_row = torch.randperm(rows * k, generator=gen, device="cuda").to(torch.int32)
    out = be.scatter_rows(src, hit_row, k)
    want = torch.empty_like(out)
    want[hit_row.long()] = src.repeat_interleave(k, dim=0)
    assert be.take_faults() == 0
    assert torch.equal(out, want)


def test_full_size_qknorm_rope_prefill_rows(be, ora):
    """Qwen3-32B at T=2048, 64 q + 8 kv heads of 128, fp16, the chunk's own table rows 0..2047 (the benchmark's headline
    launch of this op): a row subset against the oracle bit for bit, every row against the same row launched alone
    (batch == sequential, gpu_eligible_forward.rs:33-66), plain and with the K/V cache store fused in."""
    s = synth()
    T, n_q, n_kv, hd = 2048, 64, 8, 128
    gen = torch.Generator(device="cuda").manual_seed(4321)
    q0 = torch.randn((T, n_q * hd), generator=gen, device="cuda").half()
    k0 = torch.randn((T, n_kv * hd), generator=gen, device="cuda").half()
    v0 = torch.randn((T, n_kv * hd), generator=gen, device="cuda").half()
    g = s.rng(2, 2048)
    qw, kw = s.normal_f32(g, hd, 1.0, 0.05), s.normal_f32(g, hd, 1.0, 0.05)
    ropes = ora.rope_table(list(range(T)), ora.rope_inv_freq(hd, 1e6))
    dqw, dkw, dropes = dev(qw), dev(kw), dev(ropes)
    q, k = q0.clone(), k0.clone()
    be.qknorm_rope_neox(q, k, dqw, dkw, dropes, n_q, n_kv, hd, 1e-6)
    pick = [0, 1, 2, 511, 1024, 1777, 2046, 2047]
    wq, wk = host(q0[pick]).copy(), host(k0[pick]).copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, np.ascontiguousarray(ropes[pick]), 1e-6)
    assert np.array_equal(host(q[pick]), wq) and np.array_equal(host(k[pick]), wk)  # the reference's f32 result, rounded once
    for r in (0, 1000, 2047):  # a row of the batch equals the row launched alone
        q1, k1 = q0[r:r + 1].clone(), k0[r:r + 1].clone()
        be.qknorm_rope_neox(q1, k1, dqw, dkw, dropes[r:r + 1].clone(), n_q, n_kv, hd, 1e-6)
        assert torch.equal(q1[0], q[r]) and torch.equal(k1[0], k[r])
    # with the cache store: the same q and k, and the cache planes hold k (rotated) and v at the rows' positions
    pos = torch.arange(T, dtype=torch.int32, device="cuda").flip(0).contiguous()  # cache row 2047 - r
    kc = torch.zeros((T, n_kv * hd), dtype=torch.float16, device="cuda")
    vc = torch.zeros_like(kc)
    q2, k2 = q0.clone(), k0.clone()
    be.qknorm_rope_kv_store(q2, k2, v0, dqw, dkw, dropes, pos, kc, vc, n_q, n_kv, hd, 1e-6)
    assert be.take_faults() == 0
    assert torch.equal(q2, q) and torch.equal(k2, k)
    assert torch.equal(kc.flip(0), k) and torch.equal(vc.flip(0), v0)  # fp16 activations: both narrowings are the identity
    wkc, wvc = np.zeros((T, n_kv * hd), np.uint16), np.zeros((T, n_kv * hd), np.uint16)
    ora.kv_store_rows(wk, host(v0[pick]).copy(), np.array([T - 1 - r for r in pick], np.uint32), wkc, wvc)
    rows_c = [T - 1 - r for r in pick]
    assert np.array_equal(host(kc[rows_c]), wkc[rows_c]) and np.array_equal(host(vc[rows_c]), wvc[rows_c])


def test_full_size_moe_swiglu_and_prefill_swiglu_f32(be, ora):
    """The f32 SwiGLU launches of the benchmark at their exact sizes: the MoE layer's grouped [8192 x 768] (1.57 M tiles: the
    single-wave-workgroup shape of the streaming kernels, which smaller f32 cases never reach), the whole tensor against
    the oracle; and the dense prefill [2048 x 25600] on a row subset plus a relaunch of a slice."""
    gen = torch.Generator(device="cuda").manual_seed(99)
    gate = torch.randn((8192, 768), generator=gen, device="cuda")
    up = torch.randn((8192, 768), generator=gen, device="cuda")
    want = host(gate).copy()
    ora.swiglu(want.reshape(-1), host(up).reshape(-1).copy())
    be.swiglu(gate, up)
    got = host(gate)
    assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want)
    T, F = 2048, 25600
    gate = torch.randn((T, F), generator=gen, device="cuda")
    up = torch.randn((T, F), generator=gen, device="cuda")
    g0 = gate.clone()
    be.swiglu(gate, up)
    pick = [0, 1023, 2047]
    want = host(g0[pick]).copy()
    ora.swiglu(want.reshape(-1), host(up[pick]).reshape(-1).copy())
    assert rel_err_f32(host(gate[pick]), want) <= TOL_F32 and close_idiom(host(gate[pick]), want)
    part = g0[1500:1503].clone()
    be.swiglu(part, up[1500:1503].clone())
    assert torch.equal(part, gate[1500:1503])


def _device_table(rows, row_bytes, seed, tame):
    """A [rows x row_bytes] table of random bytes built on the device (nothing this size crosses the bus), its f16 scale
    fields tamed to small positive values by `tame(table)`."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    table = torch.randint(0, 256, (rows, row_bytes), generator=gen, device="cuda", dtype=torch.uint8)
    tame(table, gen)
    return table


def test_full_vocabulary_embedding_tables(be, ora):
    """The embedding gathers at the vocabulary's real size, 151 936 rows: Q8_0 [151936 x 1024] (165 MB, configs 0 and 1) and
    Q4_K [151936 x 5120] (438 MB, config 2), built on the device; ids include row 0 and row 151 935; only the gathered
    table rows come back to the host, where the oracle decodes them (QuantMat::row_into, quantmat/mod.rs:75-89)."""
    import allpaka_amd as apk

    vocab = 151936

    def tame_q8(t, gen):  # [d: f16][32 x i8] per 34 bytes: d = |N(0, 0.02)| / 127, some of them f16 subnormals
        v = t.view(vocab, -1, 34)
        d = (torch.randn((vocab, v.shape[1], 1), generator=gen, device="cuda").abs() * (0.02 / 127.0)).half()
        v[:, :, 0:2] = d.view(torch.uint8).reshape(vocab, v.shape[1], 2)

    def tame_q4k(t, gen):  # [d: f16][dmin: f16][12 scale bytes][128 nibble bytes] per 144 bytes
        v = t.view(vocab, -1, 144)
        d = (torch.randn((vocab, v.shape[1], 2), generator=gen, device="cuda").abs() * (0.02 / 63.0)).half()
        v[:, :, 0:4] = d.view(torch.uint8).reshape(vocab, v.shape[1], 4)

    g = synth().rng(0, 151936)
    for fmt_name, n_in, rb, tame, T in (("Q8_0", 1024, 1088, tame_q8, 512), ("Q4K", 5120, 2880, tame_q4k, 2048)):
        table = _device_table(vocab, rb, 7 + n_in, tame)
        ids = g.integers(0, vocab, size=T, dtype=np.uint32)
        ids[[0, 1, 2, T - 1]] = [0, vocab - 1, vocab - 1, 0]
        d_ids = dev(ids)
        qm = apk.QuantMat(be, table.view(-1), ora.FMT[fmt_name], vocab, n_in)
        for out_dtype in (torch.float32, torch.float16):
            out = torch.zeros((T, n_in), dtype=out_dtype, device="cuda")
            qm.rows_into(d_ids, out)
            picked = host(table[d_ids.long()]).reshape(-1)  # the T gathered rows as a T-row table of their own
            want = ora.embed_rows(picked, ora.FMT[fmt_name], T, n_in, np.arange(T, dtype=np.uint32), out_f16=out_dtype == torch.float16)
            assert np.array_equal(host(out), want), (fmt_name, out_dtype)
        last = ora.embed_rows(host(table[vocab - 1]).reshape(-1), ora.FMT[fmt_name], 1, n_in, np.zeros(1, np.uint32))[0]
        assert np.array_equal(host(qm.row(vocab - 1)), last)  # QuantMat::row of the table's last row
        with pytest.raises(ValueError):  # one past the table's last row: rejected on the host, as the callers reject it
            bad = ids.copy()
            bad[5] = vocab
            qm.rows_into(dev(bad), out)
        del table, qm


# ----------------------------------------------- full-size property checks
def test_full_size_prefill_properties(be, ora):
    """Qwen3-32B shapes at T=2048 (fp16): the oracle checks a row subset; the rest is
    covered by row independence (every row of a batched launch equals the same row
    launched alone, the batch==sequential property of gpu_eligible_forward.rs:33-66)."""
    s = synth()
    m = s.MODELS["qwen3-32b"]
    T, H, F = 2048, m["hidden"], m["ffn"]
    gen = torch.Generator(device="cuda").manual_seed(1234)
    x = torch.randn((T, H), generator=gen, device="cuda").half()
    d = torch.randn((T, H), generator=gen, device="cuda").half()
    gamma = (1 + 0.05 * torch.randn(H, generator=gen, device="cuda")).float()
    x0 = x.clone()
    h = torch.zeros_like(x)
    be.add_rmsnorm_rows(x, d, h, gamma, 1e-6)
    pick = [0, 1, 777, 2047]
    xs, ds = host(x0[pick]).copy(), host(d[pick]).copy()
    wh = np.zeros_like(xs)
    ora.add_rmsnorm_rows(xs, ds, wh, host(gamma), 1e-6)
    assert np.array_equal(host(x[pick]), xs) and f16_ulp_diff(host(h[pick]), wh) <= TOL_F16_ULP
    x1, h1 = x0[1000:1001].clone(), torch.zeros((1, H), dtype=torch.float16, device="cuda")
    be.add_rmsnorm_rows(x1, d[1000:1001].clone(), h1, gamma, 1e-6)
    assert torch.equal(h1[0], h[1000]) and torch.equal(x1[0], x[1000])
    # SwiGLU over [2048, 25600]: a slice against the oracle, the whole against a row-sliced relaunch
    gate = torch.randn((T, F), generator=gen, device="cuda").half()
    up = torch.randn((T, F), generator=gen, device="cuda").half()
    g0 = gate.clone()
    be.swiglu(gate, up)
    wg = host(g0[5]).copy()
    ora.swiglu(wg, host(up[5]).copy())
    assert f16_ulp_diff(host(gate[5]), wg) <= TOL_F16_ULP
    part = g0[1024:1030].clone()
    be.swiglu(part, up[1024:1030].clone())
    assert torch.equal(part, gate[1024:1030])
    # embedding gather of 2048 rows from a Q4_K table: every output row equals the single-row gather of its id
    import allpaka_amd as apk

    vocab = 4096
    table = s.q4_k_table(s.rng(2, 1), vocab, H)
    qm = apk.QuantMat(be, dev(table.reshape(-1)), ora.FMT["Q4K"], vocab, H)
    ids = s.rng(2, 2).integers(0, vocab, size=T, dtype=np.uint32)
    out = torch.zeros((T, H), dtype=torch.float16, device="cuda")
    qm.rows_into(dev(ids), out)
    sub = [0, 5, 2047]
    want = ora.embed_rows(table.reshape(-1), ora.FMT["Q4K"], vocab, H, ids[sub], out_f16=True)
    assert np.array_equal(host(out[sub]), want)
    # rows with equal ids are equal (gather idempotence)
    order = np.argsort(ids, kind="stable")
    same = [(order[i], order[i + 1]) for i in range(T - 1) if ids[order[i]] == ids[order[i + 1]]][:50]
    for a, b in same:
        assert torch.equal(out[a], out[b])


def test_stats_count_calls_and_dispatches(be):
    c0, d0, _, _ = be.stats()
    a = torch.ones(4096, device="cuda")
    be.swiglu(a, torch.ones(4096, device="cuda"))
    c1, d1, enc, wait = be.stats()
    assert c1 == c0 + 1 and d1 == d0 + 1 and enc > 0 and wait > 0

"""Tensors of more than 2^32 bytes / 2^31 elements: the index arithmetic of the streaming kernels is
64-bit.  Inputs are generated on the device; slices from the start, the 2^31- and 2^32-byte marks and the
very end are compared with the oracle."""
import numpy as np
import pytest

from util import f16_ulp_diff

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def be():
    import allpaka_amd

    b = allpaka_amd.Backend(0)
    yield b
    b.close()


def bits(t):
    return t.detach().cpu().numpy().view(np.uint16)


def test_streams_past_four_gigabytes(be, ora):
    n = (1 << 31) + (1 << 20) + 24  # fp16 elements: 4 GiB + 2 MiB + 48 bytes per tensor
    gen = torch.Generator(device="cuda").manual_seed(11)
    gate = torch.empty(n, dtype=torch.float16, device="cuda")
    up = torch.empty(n, dtype=torch.float16, device="cuda")
    step = 1 << 28
    for i in range(0, n, step):  # filled in pieces: no 8 GiB float32 temporary
        m = min(step, n - i)
        gate[i:i + m] = torch.randn(m, generator=gen, device="cuda", dtype=torch.float32).half()
        up[i:i + m] = torch.randn(m, generator=gen, device="cuda", dtype=torch.float32).half()
    windows = [(0, 4096), ((1 << 30) - 2048, 4096), ((1 << 31) - 2048, 4096), (n - 4096, 4096)]
    before = [(bits(gate[a:a + m]).copy(), bits(up[a:a + m]).copy()) for a, m in windows]
    be.swiglu(gate, up)
    for (a, m), (g0, u0) in zip(windows, before):
        want = g0.copy()
        ora.swiglu(want, u0)
        assert f16_ulp_diff(bits(gate[a:a + m]), want) <= 2, a
        assert np.array_equal(bits(up[a:a + m]), u0)
    # residual add in place over the same tensors: exact
    before = [(bits(gate[a:a + m]).copy(), bits(up[a:a + m]).copy()) for a, m in windows]
    be.add_assign_slice(gate, up)
    for (a, m), (g0, u0) in zip(windows, before):
        want = ora.f32_to_f16_bits(ora.f16_bits_to_f32(g0) + ora.f16_bits_to_f32(u0))
        assert np.array_equal(bits(gate[a:a + m]), want), a
    # GeGLU over the same tensors
    before = [(bits(gate[a:a + m]).copy(), bits(up[a:a + m]).copy()) for a, m in windows]
    be.geglu_tanh(gate, up)
    for (a, m), (g0, u0) in zip(windows, before):
        want = g0.copy()
        ora.geglu_tanh(want, u0)
        ok = (np.abs(ora.f16_bits_to_f32(bits(gate[a:a + m])) - ora.f16_bits_to_f32(want)) <= 1e-3 * (1 + np.abs(ora.f16_bits_to_f32(want))))
        assert ok.all(), a
    # a per-row bias over rows of 16 384 (131 080 rows: past 2^32 bytes), in place, bit for bit
    width = 16384
    nrows = n // width
    bias = torch.randn(width, generator=gen, device="cuda")
    before = [bits(gate[a:a + m]).copy() for a, m in windows[:3]]
    be.add_bias_rows(gate[: nrows * width], bias)
    hb = bias.cpu().numpy()
    for (a, m), g0 in zip(windows[:3], before):
        w = ora.f16_bits_to_f32(g0)
        w += hb[(np.arange(a, a + m)) % width]
        assert np.array_equal(bits(gate[a:a + m]), ora.f32_to_f16_bits(w)), a
    # fp16 -> f32 of the first 2^30 + 2^20 elements (a 4 GiB + 4 MiB result) and back
    m32 = (1 << 30) + (1 << 20)
    wide = be.cast(up[:m32], torch.float32)
    for a in (0, (1 << 29) - 2048, (1 << 30) - 2048, m32 - 4096):
        assert np.array_equal(wide[a:a + 4096].cpu().numpy().view(np.uint32), ora.f16_bits_to_f32(bits(up[a:a + 4096])).view(np.uint32)), a
    back = be.cast(wide, torch.float16)
    assert torch.equal(back, up[:m32])
    del wide, back
    # rows x n beyond 2^32 bytes: residual add + RMSNorm over 131 080 rows of 16 384 (the same memory, reshaped)
    rows, width = 131080, 16384
    x = gate[: rows * width].view(rows, width)
    d = up[: rows * width].view(rows, width)
    h = torch.empty_like(x)
    gamma = torch.ones(width, device="cuda")
    pick = [0, 1, 65535, 65536, 131071, 131072, 131079]
    before = [(bits(x[r]).copy(), bits(d[r]).copy()) for r in pick]
    be.add_rmsnorm_rows(x, d, h, gamma, 1e-6)
    for r, (x0, d0) in zip(pick, before):
        wx, wh = x0.reshape(1, -1).copy(), np.zeros((1, width), np.uint16)
        ora.add_rmsnorm_rows(wx, d0.reshape(1, -1), wh, np.ones(width, np.float32), 1e-6)
        assert np.array_equal(bits(x[r]), wx[0]), r
        assert f16_ulp_diff(bits(h[r]), wh[0]) <= 2, r
    assert be.take_faults() == 0


def test_head_rows_and_permuted_rows_past_four_gigabytes(be, ora):
    from allpaka_amd import synth as s

    # QK-norm + RoPE over q of 262 200 rows x 64 heads x 128 (4.3 GB of fp16)
    rows, n_q, n_kv, hd = 262200, 64, 1, 128
    gen = torch.Generator(device="cuda").manual_seed(5)
    q = torch.empty((rows, n_q * hd), dtype=torch.float16, device="cuda")
    for i in range(0, rows, 32768):
        m = min(32768, rows - i)
        q[i:i + m] = torch.randn((m, n_q * hd), generator=gen, device="cuda", dtype=torch.float32).half()
    k = torch.randn((rows, n_kv * hd), generator=gen, device="cuda", dtype=torch.float32).half()
    g = s.rng(3, 9)
    qw, kw = s.normal_f32(g, hd, 1.0, 0.05), s.normal_f32(g, hd, 1.0, 0.05)
    inv = ora.rope_inv_freq(hd, 1e6)
    pos = torch.arange(rows, dtype=torch.int32, device="cuda") % 32768
    table = be.rope_table(pos, torch.from_numpy(inv).cuda())
    pick = [0, 1, 131071, 131072, 262143, 262144, rows - 1]
    before = [(bits(q[r]).copy(), bits(k[r]).copy()) for r in pick]
    be.qknorm_rope_neox(q, k, torch.from_numpy(qw).cuda(), torch.from_numpy(kw).cuda(), table, n_q, n_kv, hd, 1e-6)
    for r, (q0, k0) in zip(pick, before):
        wq, wk = q0.reshape(1, -1).copy(), k0.reshape(1, -1).copy()
        ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, table[r:r + 1].cpu().numpy(), 1e-6)
        assert np.array_equal(bits(q[r]), wq[0]) and np.array_equal(bits(k[r]), wk[0]), r
    del q, k, table
    # the permuted rows [T*k, 2048] f32 beyond 4 GiB: T = 65 552 tokens, k = 8 (524 416 rows of 8 KiB)
    T, kk, cols = 65552, 8, 2048
    hs = torch.randn((T, cols), generator=gen, device="cuda")
    # a valid CSR by construction: row of hit j of token t is j*T + t (expert-major, token-ascending)
    hit_row = (torch.arange(kk, device="cuda", dtype=torch.int64)[None, :] * T + torch.arange(T, device="cuda", dtype=torch.int64)[:, None])
    hit_row = hit_row.to(torch.int32).contiguous()
    tok = torch.arange(T, device="cuda", dtype=torch.int32).repeat(kk).contiguous()
    xs = be.scatter_rows(hs, hit_row.view(-1), kk)
    for r in (0, T - 1, T, 3 * T + 77, 524287, 524288, T * kk - 1):  # 524 288 rows * 8 KiB = 4 GiB
        assert torch.equal(xs[r], hs[r % T]), r
    xg = be.gather_rows(hs, tok)
    for r in (0, T - 1, T, 3 * T + 77, 524287, 524288, T * kk - 1):
        assert torch.equal(xg[r], hs[r % T]), r
    del xg
    # the combine over the same 4.3 GB of rows (its hits past the 4 GiB mark are those of expert 7 for tokens >= 65 424):
    # x += sum of hit_w * flat[hit_row], then the norm -- chosen tokens against the oracle on their own eight rows
    flat = torch.randn((T * kk, cols), generator=gen, device="cuda")
    hit_w = torch.rand((T, kk), generator=gen, device="cuda")
    x = torch.randn((T, cols), generator=gen, device="cuda")
    hb = torch.empty_like(x)
    gamma = (1 + 0.05 * torch.randn(cols, generator=gen, device="cuda")).contiguous()
    picks = [0, 1, 65423, 65424, 65425, T - 1]
    before = {t: x[t].cpu().numpy().copy() for t in picks}
    tok_off = (torch.arange(T + 1, device="cuda", dtype=torch.int32) * kk).contiguous()
    be.moe_combine_add_rmsnorm(x, flat, tok_off, hit_row.view(-1), hit_w.view(-1), hb, gamma, 1e-6)
    for t in picks:
        rows_t = hit_row[t].cpu().numpy().astype(np.int64)
        wx = before[t].reshape(1, -1).copy()
        wh = np.zeros_like(wx)
        small = np.stack([flat[int(r)].cpu().numpy() for r in rows_t])
        ora.moe_combine_add_rmsnorm(wx, small, np.array([0, kk], np.uint32), np.arange(kk, dtype=np.uint32),
                                    hit_w[t].cpu().numpy().copy(), wh, gamma.cpu().numpy(), 1e-6)
        assert np.array_equal(x[t].cpu().numpy().view(np.uint32), wx[0].view(np.uint32)), t
        assert np.allclose(hb[t].cpu().numpy(), wh[0], rtol=1e-5, atol=1e-6), t
    assert be.take_faults() == 0


@pytest.mark.parametrize("fmt_name", ["Q4K", "Q6K", "Q8_0", "F16"])
def test_embedding_rows_past_four_gigabytes_of_output(be, ora, fmt_name):
    """420 000 gathered rows of 5120 fp16 columns are 4.3 GB of output: rows from the start, the 2^31- and 2^32-byte
    marks and the very end against the oracle (a format of each kernel family: the hand-laid Q4_K kernel, the
    super-block kernels whose lanes are numbered across the batch, the four-tiles-per-lane kernels, the staged ones)."""
    fmt, vocab, hidden, T = ora.FMT[fmt_name], 600, 5120, 420000
    rb = ora.expected_bytes(fmt, hidden)
    g = np.random.default_rng(fmt)
    raw = g.integers(0, 256, size=vocab * rb, dtype=np.uint8)
    offs = {"Q4K": (144, [0, 2]), "Q6K": (210, [208]), "Q8_0": (34, [0])}.get(fmt_name)
    if offs:
        for o in offs[1]:
            raw.reshape(-1, offs[0])[:, o + 1] &= 0x3B  # finite, small f16 scale fields
    else:
        raw.view(np.uint16)[:] &= np.uint16(0xBFFF)
    ids = g.integers(0, vocab, size=T, dtype=np.uint32)
    out = torch.empty((T, hidden), dtype=torch.float16, device="cuda")
    table = torch.from_numpy(raw).cuda()
    rc = be.L.apk_embed_rows(be.h, fmt, table.data_ptr(), vocab, hidden, torch.from_numpy(ids.view(np.int32)).cuda().data_ptr(), T,
                             out.data_ptr(), 1)
    assert rc == 0
    be.sync()
    per_row = hidden * 2
    pick = sorted({0, 1, (1 << 31) // per_row - 1, (1 << 31) // per_row, (1 << 31) // per_row + 1, (1 << 32) // per_row - 1,
                   (1 << 32) // per_row, (1 << 32) // per_row + 1, T - 2, T - 1})
    want = ora.embed_rows(raw, fmt, vocab, hidden, ids[pick], out_f16=True)
    for i, r in enumerate(pick):
        assert np.array_equal(bits(out[r]), want[i].view(np.uint16)), (fmt_name, r)
    assert be.take_faults() == 0

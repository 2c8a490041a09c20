"""Seeded random shapes for every op through the C ABI against the CPU oracle.

The parametrised parity tests pin the benchmark shapes and hand-picked edges; this
file draws the shapes (row counts, row lengths, head geometry, expert counts, top-k,
formats) from a fixed-seed generator so that indexing that only breaks off the
beaten path (a last partial tile, a workgroup tail, a wave that owns no head) is met
too.  Same bars: bit-exact for integer / byte / index work and pure data movement,
1e-5 relative for f32, 2 ulp for fp16.
"""
import os

import numpy as np
import pytest

from util import close_idiom, f16_ulp_diff, rel_err_f32

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

TOL_F32 = 1e-5
TOL_F16_ULP = 2
CASES = int(os.environ.get("APK_RANDOM_CASES", "24"))  # more cases for an occasional wider run


@pytest.fixture(scope="module")
def be():
    import allpaka_amd

    b = allpaka_amd.Backend(0)
    yield b
    b.close()


def dev(a):
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


def S():
    from allpaka_amd import synth

    return synth


def act(g, shape, f16):
    a = S().normal_f32(g, shape)
    return S().to_f16_bits(a) if f16 else a


def check_float(got, want, f16, what):
    if f16:
        assert f16_ulp_diff(got, want) <= TOL_F16_ULP, what
    else:
        assert rel_err_f32(got, want) <= TOL_F32 and close_idiom(got, want), what


@pytest.mark.parametrize("case", range(CASES))
def test_add_rmsnorm_random(be, ora, case):
    g = np.random.default_rng(1000 + case)
    f16 = bool(case & 1)
    rows = int(g.integers(1, 70))
    n = int(g.integers(1, 1300)) * 8 if case % 3 else int(g.integers(1, 9000))  # every third case: a ragged row length
    x, d = act(g, (rows, n), f16), act(g, (rows, n), f16)
    gamma = S().normal_f32(g, n, 1.0, 0.05)
    with_delta = case % 4 != 3
    wx, wh = x.copy(), np.zeros_like(x)
    ora.add_rmsnorm_rows(wx, d if with_delta else None, wh, gamma, 1e-6)
    tx, th = dev(x), torch.zeros_like(dev(x))
    be.add_rmsnorm_rows(tx, dev(d) if with_delta else None, th, dev(gamma), 1e-6)
    assert np.array_equal(host(tx), wx), (rows, n, f16)  # the residual sum is exact
    check_float(host(th), wh, f16, (rows, n, f16))


@pytest.mark.parametrize("case", range(12))
def test_add_rmsnorm_random_batches(be, ora, case):
    """Row counts in the thousands: the launch shapes the host picks by batch size (a wave per row while the
    batch is resident at once, two tiles per lane beyond, four rows per workgroup from 8192 rows on)."""
    g = np.random.default_rng(1500 + case)
    f16 = bool(case & 1)
    n = int(g.integers(8, 770)) * 8
    rows = int(g.integers(1000, min(9000, 12_000_000 // n) + 1))
    x, d = act(g, (rows, n), f16), act(g, (rows, n), f16)
    gamma = S().normal_f32(g, n, 1.0, 0.05)
    wx, wh = x.copy(), np.zeros_like(x)
    ora.add_rmsnorm_rows(wx, d, wh, gamma, 1e-6)
    tx, th = dev(x), torch.zeros_like(dev(x))
    be.add_rmsnorm_rows(tx, dev(d), th, dev(gamma), 1e-6)
    assert np.array_equal(host(tx), wx), (rows, n, f16)
    check_float(host(th), wh, f16, (rows, n, f16))


@pytest.mark.parametrize("case", range(CASES))
def test_postnorm_add_rmsnorm_random(be, ora, case):
    """The sandwich norm and the next norm in one call, over drawn row counts and lengths (tiled kernels, ragged and
    short rows): against the oracle's two norms and the add between them."""
    g = np.random.default_rng(1700 + case)
    f16 = bool(case & 1)
    if case % 4 == 3:  # batches in the thousands
        n = int(g.integers(8, 500)) * 8
        rows = int(g.integers(1000, min(6000, 6_000_000 // n) + 1))
    else:
        rows = int(g.integers(1, 70))
        n = int(g.integers(1, 1300)) * 8 if case % 3 else int(g.integers(1, 9000))
    x, d = act(g, (rows, n), f16), act(g, (rows, n), f16)
    pg, gamma = S().normal_f32(g, n, 1.0, 0.05), S().normal_f32(g, n, 1.0, 0.05)
    nd = np.zeros_like(d)
    ora.add_rmsnorm_rows(d.copy(), None, nd, pg, 1e-6)
    wx, wh = x.copy(), np.zeros_like(x)
    ora.add_rmsnorm_rows(wx, nd, wh, gamma, 1e-6)
    tx, th = dev(x), torch.zeros_like(dev(x))
    be.postnorm_add_rmsnorm_rows(tx, dev(d), dev(pg), th, dev(gamma), 1e-6)
    what = (rows, n, f16)
    if f16:
        # the sum can cancel: held to 2 ulp, or to one ulp of its larger operand where the two-step path's
        # normalised delta is an ulp off
        fv = lambda a: a.view(np.float16).astype(np.float64)  # noqa: E731
        key = lambda b: np.where(b.astype(np.int32) & 0x8000, 0x8000 - b.astype(np.int32), b.astype(np.int32))  # noqa: E731
        slack = 2.0 ** -10 * np.maximum(np.abs(fv(x)), np.abs(fv(nd)))
        gx = host(tx)
        assert np.all((np.abs(key(gx) - key(wx)) <= TOL_F16_ULP) | (np.abs(fv(gx) - fv(wx)) <= slack)), what
        assert np.mean(gx == wx) > 0.99, what
        assert np.mean(np.abs(key(host(th)) - key(wh)) <= TOL_F16_ULP) > 0.999, what
    else:
        check_float(host(tx), wx, False, what)
        check_float(host(th), wh, False, what)


@pytest.mark.parametrize("case", range(CASES))
def test_attn_prologue_random(be, ora, case):
    """Projection biases (any subset), per-head norms (any subset), either pairing, drawn head geometry, with and
    without the K/V cache store, against the oracle's ops in the reference's order (attention.rs:125-165, kv.rs:682-697)."""
    g = np.random.default_rng(2600 + case)
    f16 = bool(case & 1)
    rows = int(g.integers(1, 60)) if case % 6 else int(g.integers(1500, 2600))
    n_q, n_kv = int(g.integers(1, 40)), int(g.integers(1, 9))
    hd = int(g.choice([64, 128, 256]))
    if hd == 256 or rows > 1000:
        n_q = min(n_q, 12)
    style = int(g.integers(0, 2))
    es = 2 if f16 else 4
    tile = 16 // es if style else 2 * (16 // es)  # rotary widths the tiled kernels take
    rot = hd if case % 3 else int(g.integers(1, hd // tile + 1)) * tile
    store = case % 4 != 3
    q, k, v = act(g, (rows, n_q * hd), f16), act(g, (rows, n_kv * hd), f16), act(g, (rows, n_kv * hd), f16)
    qb = S().normal_f32(g, n_q * hd, 0.0, 0.5) if case % 5 else None
    kb = S().normal_f32(g, n_kv * hd, 0.0, 0.5) if case % 7 else None
    vb = S().normal_f32(g, n_kv * hd, 0.0, 0.5) if case % 2 or case % 3 else None
    qw = S().normal_f32(g, hd, 1.0, 0.05) if case % 4 < 2 else None
    kw = S().normal_f32(g, hd, 1.0, 0.05) if case % 4 in (0, 3) else None
    cap = rows + 11
    positions = g.permutation(cap)[:rows].astype(np.uint32)
    ropes = ora.rope_table([int(p) for p in positions], ora.rope_inv_freq(rot, 1e6))
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6, style=style, q_bias=qb, k_bias=kb)
    wv = v
    if vb is not None:
        wv = ora.f16_bits_to_f32(v) if f16 else v.copy()
        ora.add_bias_rows(wv, vb)
        wv = ora.f32_to_f16_bits(wv) if f16 else wv
    wkc, wvc = np.zeros((cap, n_kv * hd), np.uint16), np.zeros((cap, n_kv * hd), np.uint16)
    ora.kv_store_rows(wk, wv, positions, wkc, wvc)
    tq, tk, tv = dev(q), dev(k), dev(v)
    kc = torch.zeros((cap, n_kv * hd), dtype=torch.float16, device="cuda")
    vc = torch.zeros_like(kc)
    d = lambda a: None if a is None else dev(a)  # noqa: E731
    kwargs = dict(q_bias=d(qb), k_bias=d(kb), v_bias=d(vb), q_norm=d(qw), k_norm=d(kw), adjacent_pairs=bool(style), rot_dim=rot)
    if store:
        kwargs.update(cache_pos=dev(positions), k_cache=kc, v_cache=vc)
    be.attn_prologue_rows(tq, tk, tv, n_q, n_kv, hd, 1e-6, dev(ropes), **kwargs)
    what = (rows, n_q, n_kv, hd, rot, style, f16, store, qb is not None, kb is not None, vb is not None)
    gk = host(tk)
    check_float(host(tq), wq, f16, what)
    check_float(gk, wk, f16, what)
    assert np.array_equal(host(tv), wv), what
    if store:
        assert np.array_equal(host(vc), wvc), what
        mine_k, mine_v = np.zeros_like(wkc), np.zeros_like(wvc)
        ora.kv_store_rows(gk, wv, positions, mine_k, mine_v)
        assert np.array_equal(host(kc), mine_k), what
        assert f16_ulp_diff(host(kc), wkc) <= (TOL_F16_ULP if f16 else 1), what


@pytest.mark.parametrize("case", range(CASES))
def test_qknorm_rope_random(be, ora, case):
    g = np.random.default_rng(2000 + case)
    f16 = bool(case & 1)
    rows = int(g.integers(1, 40))
    n_q, n_kv = int(g.integers(0, 70)), int(g.integers(0, 12))
    if n_q + n_kv == 0:
        n_q = 1
    if case % 3:  # the tiled kernels
        hd = int(g.choice([64, 128, 256]))
        rot, style = hd, 0
    else:  # the element-wise kernel: any geometry
        hd = int(g.integers(1, 160)) * 2
        rot = int(g.integers(0, hd // 2 + 1)) * 2
        style = int(g.integers(0, 2))
    if hd == 256:
        n_q = min(n_q, 24)
    q, k = act(g, (rows, n_q * hd), f16), act(g, (rows, n_kv * hd), f16)
    qw = S().normal_f32(g, hd, 1.0, 0.05) if case % 5 else None
    kw = S().normal_f32(g, hd, 1.0, 0.05) if case % 7 else None
    positions = [int(v) for v in g.integers(0, 32768, size=rows)]
    ropes = ora.rope_table(positions, ora.rope_inv_freq(rot, 1e6)) if rot else np.zeros((rows, 0, 2), np.float32)
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6, style=style)
    tq, tk = dev(q), dev(k)
    fn = be.qknorm_rope_norm if style else be.qknorm_rope_neox
    rt = dev(ropes) if rot else torch.zeros((rows, 0, 2), device="cuda")
    fn(tq, tk, None if qw is None else dev(qw), None if kw is None else dev(kw), rt, n_q, n_kv, hd, 1e-6, rot_dim=rot)
    what = (rows, n_q, n_kv, hd, rot, style, f16)
    if n_q:
        check_float(host(tq), wq, f16, what)
    if n_kv:
        check_float(host(tk), wk, f16, what)


@pytest.mark.parametrize("case", range(12))
def test_qknorm_rope_random_batches(be, ora, case):
    """Prefill-sized batches of the tiled kernels: enough waves for two passes per q wave in fp16, row
    counts that are no multiple of anything."""
    g = np.random.default_rng(2500 + case)
    f16 = bool(case & 1)
    hd = int(g.choice([64, 128, 256]))
    n_q, n_kv = int(g.integers(1, 41)), int(g.integers(0, 9))
    rows = int(g.integers(200, min(3000, 10_000_000 // ((n_q + n_kv) * hd)) + 1))
    q, k = act(g, (rows, n_q * hd), f16), act(g, (rows, n_kv * hd), f16)
    qw, kw = S().normal_f32(g, hd, 1.0, 0.05), S().normal_f32(g, hd, 1.0, 0.05)
    positions = [int(v) for v in g.integers(0, 32768, size=rows)]
    ropes = ora.rope_table(positions, ora.rope_inv_freq(hd, 1e6))
    wq, wk = q.copy(), k.copy()
    ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ropes, 1e-6)
    tq, tk = dev(q), dev(k)
    be.qknorm_rope_neox(tq, tk, dev(qw), dev(kw), dev(ropes), n_q, n_kv, hd, 1e-6)
    what = (rows, n_q, n_kv, hd, f16)
    check_float(host(tq), wq, f16, what)
    if n_kv:
        check_float(host(tk), wk, f16, what)
    if f16:  # the definition, bit for bit
        assert np.array_equal(host(tq), wq), what


@pytest.mark.parametrize("case", range(CASES))
def test_swiglu_and_add_assign_random(be, ora, case):
    g = np.random.default_rng(3000 + case)
    f16 = bool(case & 1)
    n = int(g.integers(1, 200000))
    gate, up = act(g, n, f16), act(g, n, f16)
    want = gate.copy()
    ora.swiglu(want, up)
    tg, tu = dev(gate), dev(up)
    be.swiglu(tg, tu)
    check_float(host(tg), want, f16, (n, f16))
    assert np.array_equal(host(tu), up)
    ta = dev(gate)
    be.add_assign_slice(ta, tu)
    if f16:
        want = ora.f32_to_f16_bits(ora.f16_bits_to_f32(gate) + ora.f16_bits_to_f32(up))
    else:
        want = gate + up
    assert np.array_equal(host(ta), want), (n, f16)


_FORMATS = ["Q4K", "Q5K", "Q6K", "Q8_0", "Q2K", "Q3K", "Q5_0", "F16", "F32", "BF16"]
_SCALE_OFFS = {"Q4K": (144, (0, 2)), "Q5K": (176, (0, 2)), "Q6K": (210, (208,)), "Q8_0": (34, (0,)), "Q2K": (84, (80, 82)),
               "Q3K": (110, (108,)), "Q5_0": (22, (0,))}


@pytest.mark.parametrize("case", range(CASES))
def test_embed_rows_random(be, ora, case):
    import allpaka_amd as apk

    g = np.random.default_rng(4000 + case)
    name = _FORMATS[case % len(_FORMATS)]
    fmt = ora.FMT[name]
    block = {"Q8_0": 32, "Q5_0": 32, "F16": 8, "F32": 8, "BF16": 8}.get(name, 256)
    n_in = block * int(g.integers(1, 9 if block == 256 else 40))
    vocab, t = int(g.integers(1, 50)), int(g.integers(1, 60))
    rb = ora.expected_bytes(fmt, n_in)
    raw = g.integers(0, 256, size=vocab * rb, dtype=np.uint8)
    if name in _SCALE_OFFS:  # keep the f16 scale fields finite and small
        bb, offs = _SCALE_OFFS[name]
        blocks = raw.reshape(-1, bb)
        for o in offs:
            blocks[:, o + 1] &= 0x3B
    elif name == "F32":
        raw = S().normal_f32(g, vocab * n_in).view(np.uint8).copy()
    else:
        raw.view(np.uint16)[:] &= np.uint16(0xBFFF)
    ids = g.integers(0, vocab, size=t, dtype=np.uint32)
    out_f16 = bool(case & 1)
    scale = 1.0 if case % 3 else 1.7320508
    want = ora.embed_rows(raw, fmt, vocab, n_in, ids, out_f16=out_f16, scale=scale)
    qm = apk.QuantMat(be, dev(raw), fmt, vocab, n_in)
    out = torch.zeros((t, n_in), dtype=torch.float16 if out_f16 else torch.float32, device="cuda")
    qm.rows_into(dev(ids), out, embed_scale=scale)
    got = host(out)
    v = np.uint16 if out_f16 else np.uint32
    assert np.array_equal(got.view(v), want.view(v)), (name, n_in, vocab, t, out_f16, scale)


@pytest.mark.parametrize("case", range(CASES))
def test_moe_chain_random(be, ora, case):
    """router -> grouping -> permute (both forms) -> combine + residual + norm on one random shape"""
    g = np.random.default_rng(5000 + case)
    f16 = bool(case & 1)
    rows = int(g.integers(1, 300))
    n_expert = int(g.integers(1, 1025)) if case % 4 == 0 else int(g.integers(1, 257))
    k = int(g.integers(1, min(n_expert, 16) + 1))
    n = int(g.integers(1, 260)) * 8
    logits = S().normal_f32(g, (rows, n_expert))
    norm, scale = bool(case % 3), 1.0 + 0.5 * (case % 2)
    want_ids, want_w = ora.route_rows(logits, k, ora.SOFTMAX, norm, scale, threads=4)
    ids, w = be.route_rows(dev(logits), k, norm=norm, scale=scale)
    assert np.array_equal(host(ids), want_ids), (rows, n_expert, k)
    assert np.array_equal(host(w), want_w)  # the router's scores are the reference's bit for bit
    # from here on, the oracle's picks (identical ids; weights equal to 1e-5 would blur the bit-exact checks)
    want = ora.moe_group(want_ids, want_w, n_expert)
    got = be.moe_permute(dev(want_ids), dev(want_w), n_expert)
    for name, a, b in zip(["table", "tok", "tok_off", "hit_row", "hit_w"], got, want):
        assert np.array_equal(host(a).view(np.uint32), b.view(np.uint32)), (name, rows, n_expert, k)
    table, tok, tok_off, hit_row, hit_w = want
    hs = act(g, (rows, n), f16)
    xe = be.gather_rows(dev(hs), got[1])
    assert np.array_equal(host(xe), ora.gather_rows(hs, tok))
    assert torch.equal(be.scatter_rows(dev(hs), got[3], k), xe)
    flat, x = act(g, (rows * k, n), f16), act(g, (rows, n), f16)
    gamma = S().normal_f32(g, n, 1.0, 0.05)
    wx, wh = x.copy(), np.zeros_like(x)
    ora.moe_combine_add_rmsnorm(wx, flat, tok_off, hit_row, hit_w, wh, gamma, 1e-6)
    tx, th = dev(x), torch.zeros_like(dev(x))
    be.moe_combine_add_rmsnorm(tx, dev(flat), got[2], got[3], got[4], th, dev(gamma), 1e-6)
    assert np.array_equal(host(tx), wx), (rows, k, n, f16)
    check_float(host(th), wh, f16, (rows, k, n, f16))


@pytest.mark.parametrize("case", range(CASES))
def test_argmax_and_softmax_random(be, ora, case):
    g = np.random.default_rng(6000 + case)
    rows, n = int(g.integers(1, 80)), int(g.integers(1, 40000))
    logits = S().normal_f32(g, (rows, n))
    if n > 3:  # exact ties: the last maximum wins
        r, a, b = int(g.integers(0, rows)), int(g.integers(0, n)), int(g.integers(0, n))
        logits[r, a] = logits[r, b] = 9.5
    want = np.array([ora.argmax_last(r_) for r_ in logits], np.uint32)
    assert np.array_equal(host(be.argmax_rows(dev(logits))), want), (rows, n)
    m = min(n, 4096)
    x = np.ascontiguousarray(logits[:, :m])
    wsm = x.copy()
    for r_ in wsm:
        ora.softmax(r_)
    t = dev(x)
    be.softmax(t)
    assert rel_err_f32(host(t), wsm) <= TOL_F32, (rows, m)

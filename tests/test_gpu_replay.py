"""Record / replay of op chains (apk_capture_* / apk_graph_*) through the C ABI.

A replay must produce exactly what the same chain produces when run op by op
(same kernels, same launch shapes: bit-identical), and that in turn is checked
against the CPU oracle to the bars of the parity tests.  Every graph is replayed
several times with unrecorded work and waits between the replays, and every
replay is checked.
"""
import numpy as np
import pytest

from util import f16_ulp_diff, rel_err_f32

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

CAPTURE = 7  # APK_DECLINE_CAPTURE


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


class Chain:
    """The decode chain of one layer on fixed buffers: residual add + RMSNorm, QK-norm + RoPE,
    residual add + RMSNorm, SwiGLU, then the greedy argmax over a logits block."""

    def __init__(self, rows, f16, seed):
        from allpaka_amd import synth as s

        g = s.rng(3, seed)
        self.rows, self.f16 = rows, f16
        self.H, self.nq, self.nkv, self.hd, self.F, self.V = 1024, 16, 8, 128, 3072, 5000
        dt = np.float16 if f16 else np.float32

        def act(*shape):
            a = g.standard_normal(shape, dtype=np.float32).astype(dt)
            return a.view(np.uint16) if f16 else a

        self.src = {
            "x": act(rows, self.H), "d1": act(rows, self.H), "d2": act(rows, self.H),
            "q": act(rows, self.nq * self.hd), "k": act(rows, self.nkv * self.hd),
            "gate": act(rows, self.F), "up": act(rows, self.F),
            "logits": g.standard_normal((rows, self.V), dtype=np.float32),
        }
        self.g1 = (1 + 0.05 * g.standard_normal(self.H, dtype=np.float32)).astype(np.float32)
        self.g2 = (1 + 0.05 * g.standard_normal(self.H, dtype=np.float32)).astype(np.float32)
        self.qw = (0.88 + 0.001 * np.arange(self.hd)).astype(np.float32)
        self.kw = (0.92 + 0.001 * np.arange(self.hd)).astype(np.float32)
        self.pos = g.integers(0, 32768, size=rows, dtype=np.uint32)
        self.eps = 1e-6
        # device side: pristine copies + the working buffers the graph bakes in
        self.pristine = {k: dev(v) for k, v in self.src.items()}
        self.buf = {k: torch.empty_like(v) for k, v in self.pristine.items()}
        self.h1 = torch.empty_like(self.buf["x"])
        self.h2 = torch.empty_like(self.buf["x"])
        self.out = torch.zeros(rows, dtype=torch.int32, device="cuda")
        self.dg1, self.dg2, self.dqw, self.dkw = dev(self.g1), dev(self.g2), dev(self.qw), dev(self.kw)

    def rope(self, be, ora):
        inv = ora.rope_inv_freq(self.hd, 1e6)
        self.table = ora.rope_table(self.pos, inv)
        self.dtable = dev(self.table)

    def reset(self):
        for k, v in self.pristine.items():
            self.buf[k].copy_(v)
        self.h1.zero_()
        self.h2.zero_()
        self.out.zero_()
        torch.cuda.synchronize()

    def run(self, be):
        b = self.buf
        be.add_rmsnorm_rows(b["x"], b["d1"], self.h1, self.dg1, self.eps)
        be.qknorm_rope_neox(b["q"], b["k"], self.dqw, self.dkw, self.dtable, self.nq, self.nkv, self.hd, self.eps)
        be.add_rmsnorm_rows(b["x"], b["d2"], self.h2, self.dg2, self.eps)
        be.swiglu(b["gate"], b["up"])
        be.argmax_rows_into(b["logits"], self.out)

    def snapshot(self, be):
        be.sync()
        return {k: host(t).copy() for k, t in
                dict(x=self.buf["x"], h1=self.h1, h2=self.h2, q=self.buf["q"], k=self.buf["k"],
                     gate=self.buf["gate"], out=self.out).items()}

    def oracle(self, ora):
        s = {k: v.copy() for k, v in self.src.items()}
        h1 = np.zeros_like(s["x"])
        h2 = np.zeros_like(s["x"])
        ora.add_rmsnorm_rows(s["x"], s["d1"], h1, self.g1, self.eps)
        ora.qknorm_rope_rows(s["q"], s["k"], self.nq, self.nkv, self.hd, self.qw, self.kw, self.table, self.eps)
        ora.add_rmsnorm_rows(s["x"], s["d2"], h2, self.g2, self.eps)
        ora.swiglu(s["gate"], s["up"])
        out = np.array([ora.argmax_last(r) for r in s["logits"]], np.uint32)
        return dict(x=s["x"], h1=h1, h2=h2, q=s["q"], k=s["k"], gate=s["gate"], out=out)


def same_bits(a, b):
    return all(np.array_equal(a[k].view(np.uint8), b[k].view(np.uint8)) for k in a)


@pytest.mark.parametrize("rows,f16", [(1, False), (6, True), (64, True)])
def test_replay_equals_eager_and_oracle(be, ora, rows, f16):
    ch = Chain(rows, f16, 100 + rows)
    ch.rope(be, ora)
    ch.reset()
    ch.run(be)  # unrecorded first: settles the argmax scratch
    eager = ch.snapshot(be)
    want = ch.oracle(ora)
    assert np.array_equal(eager["out"], want["out"])
    for key in ("x", "h1", "h2", "q", "k", "gate"):
        if f16:
            assert f16_ulp_diff(eager[key], want[key]) <= 2, key
        else:
            assert rel_err_f32(eager[key], want[key]) <= 1e-5, key

    ch.reset()
    with be.record() as rec:
        ch.run(be)
    g = rec.graph
    assert g.nodes == 5
    # nothing ran while recording
    be.sync()
    assert np.array_equal(host(ch.buf["x"]), ch.src["x"])
    d0 = be.stats()[1]
    for rep in range(4):
        ch.reset()
        g.launch()
        got = ch.snapshot(be)
        assert same_bits(got, eager), f"replay {rep}"
        # unrecorded work between replays
        be.swiglu(ch.buf["gate"], ch.buf["up"])
        be.sync()
    assert be.stats()[1] - d0 == 4 * 5 + 4
    g.destroy()


def test_back_to_back_replays_compose(be, ora):
    """Two replays without a reset run the chain twice: equal to two eager runs."""
    ch = Chain(6, False, 7)
    ch.rope(be, ora)
    ch.reset()
    ch.run(be)
    ch.run(be)
    eager2 = ch.snapshot(be)
    ch.reset()
    with be.record() as rec:
        ch.run(be)
    ch.reset()
    rec.graph.launch()
    rec.graph.launch()
    assert same_bits(ch.snapshot(be), eager2)
    rec.graph.destroy()


def test_entries_that_wait_or_allocate_decline_inside_a_recording(be):
    import ctypes as C

    import allpaka_amd as apk

    L, h = be.L, be.h
    x = torch.ones(4, 64, device="cuda")
    gamma = torch.ones(64, device="cuda")
    hbuf = torch.empty_like(x)
    host_buf = (C.c_float * 4)()
    p = C.c_void_p()
    ms = C.c_float()
    f = C.c_uint32()
    ids = (C.c_uint32 * 1)(0)
    be.capture_begin()
    try:
        assert L.apk_sync(h) == CAPTURE
        assert L.apk_malloc(h, 64, C.byref(p)) == CAPTURE and not p.value
        assert L.apk_free(h, None) == CAPTURE
        assert L.apk_h2d(h, x.data_ptr(), host_buf, 16) == CAPTURE
        assert L.apk_d2h(h, host_buf, x.data_ptr(), 16) == CAPTURE
        assert L.apk_attach(h, host_buf, 16) == CAPTURE
        assert L.apk_detach(h, host_buf) == CAPTURE
        assert L.apk_take_faults(h, C.byref(f)) == CAPTURE
        assert L.apk_timer_begin(h) == CAPTURE
        assert L.apk_timer_end(h, C.byref(ms)) == CAPTURE
        assert L.apk_embed_rows_host_ids(h, 8, x.data_ptr(), 4, 64, ids, 1, hbuf.data_ptr(), 0) == CAPTURE
        assert L.apk_capture_begin(h) == CAPTURE
        assert b"recording" in L.apk_last_error()
        # a declined entry leaves the recording intact
        be.add_rmsnorm_rows(x, None, hbuf, gamma, 0.0)
    except BaseException:
        be.capture_abort()
        raise
    g = be.capture_end()
    assert g.nodes == 1
    assert L.apk_graph_launch(h, g.g) == 0
    be.sync()
    assert torch.allclose(hbuf, torch.ones_like(hbuf))
    g.destroy()
    # outside a recording
    gp = C.c_void_p()
    assert L.apk_capture_end(h, C.byref(gp)) == CAPTURE and not gp.value
    assert L.apk_capture_abort(h) == 0
    with pytest.raises(apk.Declined):
        be.capture_end()


def test_aborted_recording_runs_nothing_and_leaves_the_stream_usable(be):
    x = torch.full((2, 64), 3.0, device="cuda")
    up = torch.full((2, 64), 2.0, device="cuda")
    be.capture_begin()
    be.swiglu(x, up)
    be.capture_abort()
    be.sync()
    assert torch.equal(x, torch.full_like(x, 3.0))
    be.swiglu(x, up)
    be.sync()
    assert not torch.equal(x, torch.full_like(x, 3.0))


def test_argmax_scratch_cannot_move_under_a_graph(be):
    import allpaka_amd as apk

    b2 = apk.Backend(0)  # fresh context: no scratch yet
    try:
        logits = torch.randn(8, 1000, device="cuda")
        out = torch.zeros(8, dtype=torch.int32, device="cuda")
        b2.capture_begin()
        with pytest.raises(apk.Declined) as e:
            b2.argmax_rows_into(logits, out)
        assert e.value.reason == CAPTURE
        b2.capture_abort()
        b2.argmax_rows_into(logits, out)  # unrecorded: allocates the scratch
        with b2.record() as rec:
            b2.argmax_rows_into(logits, out)
        big = torch.randn(1000, 16, device="cuda")
        with pytest.raises(apk.Declined) as e:
            b2.argmax_rows(big)  # would grow (and move) the scratch the graph points at
        assert e.value.reason == CAPTURE
        out.zero_()
        rec.graph.launch()
        b2.sync()
        assert torch.equal(out.long(), torch.argmax(logits, dim=1))
        rec.graph.destroy()
        assert b2.argmax_rows(big).shape[0] == 1000  # free to grow again
    finally:
        b2.close()


@pytest.mark.parametrize("f16", [False, True])
def test_one_recording_serves_every_token_of_a_decode(be, ora, f16):
    """The reference's graph-replayable decode keeps the token position in device memory
    (d_pos, gpu/cuda/runtime/device.rs:154; build_rope_freq_dpos + rmsnorm_rope_qk_store_table_dpos,
    gpu/cuda/kernels.rs:680-765).  Same here: the recorded step builds the rotary row from a position
    buffer and stores K/V at that position; between replays only the contents of buffers change."""
    from allpaka_amd import synth as s

    n_q, n_kv, hd, cap = 16, 8, 128, 64
    g = s.rng(3, 4242)
    inv = ora.rope_inv_freq(hd, 1e6)
    qw = (0.88 + 0.001 * np.arange(hd)).astype(np.float32)
    kw = (0.92 + 0.001 * np.arange(hd)).astype(np.float32)
    dt = torch.float16 if f16 else torch.float32
    tq = torch.empty((1, n_q * hd), dtype=dt, device="cuda")
    tk = torch.empty((1, n_kv * hd), dtype=dt, device="cuda")
    tv = torch.empty((1, n_kv * hd), dtype=dt, device="cuda")
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    table = torch.zeros((1, hd // 2, 2), dtype=torch.float32, device="cuda")
    kc = torch.zeros((cap, n_kv * hd), dtype=torch.float16, device="cuda")
    vc = torch.zeros((cap, n_kv * hd), dtype=torch.float16, device="cuda")
    dinv, dqw, dkw = dev(inv), dev(qw), dev(kw)
    with be.record() as rec:
        be.rope_table_into(pos, dinv, table)
        be.qknorm_rope_kv_store(tq, tk, tv, dqw, dkw, table, pos, kc, vc, n_q, n_kv, hd, 1e-6)
    assert rec.graph.nodes == 2
    want_kc, want_vc = np.zeros((cap, n_kv * hd), np.uint16), np.zeros((cap, n_kv * hd), np.uint16)
    for p in (0, 1, 17, 63, 5, 17):  # 17 twice: a position may be rewritten
        def act(n):
            a = s.normal_f32(g, (1, n))
            return s.to_f16_bits(a) if f16 else a
        q, k, v = act(n_q * hd), act(n_kv * hd), act(n_kv * hd)
        tq.copy_(dev(q)), tk.copy_(dev(k)), tv.copy_(dev(v))
        pos.fill_(p)
        torch.cuda.synchronize()
        rec.graph.launch()
        be.sync()
        assert be.take_faults() == 0
        wq, wk = q.copy(), k.copy()
        ora.qknorm_rope_rows(wq, wk, n_q, n_kv, hd, qw, kw, ora.rope_table([p], inv), 1e-6)
        if f16:
            assert f16_ulp_diff(host(tq), wq) <= 2 and f16_ulp_diff(host(tk), wk) <= 2
        else:
            assert rel_err_f32(host(tq), wq) <= 1e-5 and rel_err_f32(host(tk), wk) <= 1e-5
        # the cache holds the exact narrowing of the k this launch produced, and of v
        ora.kv_store_rows(host(tk), v, [p], want_kc, want_vc)
        assert np.array_equal(host(kc), want_kc) and np.array_equal(host(vc), want_vc)
    # a position past the capacity: the row's store is skipped and the status word says so
    pos.fill_(cap)
    torch.cuda.synchronize()
    rec.graph.launch()
    be.sync()
    assert be.take_faults() == 8  # APK_FAULT_CACHE_RANGE
    assert np.array_equal(host(kc), want_kc)
    rec.graph.destroy()


def test_grouping_scratch_cannot_move_under_a_graph(be, ora):
    """The two-launch grouping of large batches keeps per-part counts in context scratch: same rule as the
    argmax scratch."""
    import allpaka_amd as apk
    from allpaka_amd import synth as s

    b2 = apk.Backend(0)  # fresh context: no scratch yet
    try:
        rows, k, ne = 3000, 4, 32
        logits = s.normal_f32(s.rng(4, 31), (rows, ne))
        ids, w = ora.route_rows(logits, k, threads=4)
        want = ora.moe_group(ids, w, ne)
        dids, dw = dev(ids), dev(w)
        b2.capture_begin()
        with pytest.raises(apk.Declined) as e:
            b2.moe_permute(dids, dw, ne)
        assert e.value.reason == CAPTURE
        b2.capture_abort()
        got = b2.moe_permute(dids, dw, ne)  # unrecorded: allocates the scratch
        outs = None
        with b2.record() as rec:
            outs = b2.moe_permute(dids, dw, ne)
        assert rec.graph.nodes == 2
        for t in outs:
            t.zero_()
        rec.graph.launch()
        b2.sync()
        for name, a, b in zip(["table", "tok", "tok_off", "hit_row", "hit_w"], outs, want):
            assert np.array_equal(host(a)[: b.shape[0]].view(np.uint32), b.view(np.uint32)), name
        big_ids = dev(np.zeros((9000, 4), np.uint32) + np.arange(4, dtype=np.uint32))
        with pytest.raises(apk.Declined) as e:
            b2.moe_permute(big_ids, dev(np.ones((9000, 4), np.float32)), ne)  # more parts: the scratch would move
        assert e.value.reason == CAPTURE
        rec.graph.destroy()
        assert b2.moe_permute(big_ids, dev(np.ones((9000, 4), np.float32)), ne)[1].numel() == 36000
    finally:
        b2.close()


def test_recorded_router_and_grouping_follow_the_logits_of_every_replay(be, ora):
    """The one-launch router + grouping of a decode step inside a recording: one node, and every replay
    routes the logits that are in the buffer at that time."""
    from allpaka_amd import synth as s

    rows, ne, k = 4, 128, 8
    logits = torch.zeros((rows, ne), device="cuda")
    with be.record() as rec:
        (ids, w), outs = be.route_group(logits, k)
    assert rec.graph.nodes == 1
    for step in range(4):
        fresh = s.normal_f32(s.rng(4, 700 + step), (rows, ne))
        logits.copy_(dev(fresh))
        for t in (ids, w) + tuple(outs):
            t.zero_()
        be.swiglu(torch.ones(64, device="cuda"), torch.ones(64, device="cuda"))  # unrecorded work in between
        rec.graph.launch()
        be.sync()
        o_ids, o_w = ora.route_rows(fresh, k, threads=2)
        assert np.array_equal(host(ids), o_ids) and rel_err_f32(host(w), o_w) <= 1e-5
        want = ora.moe_group(o_ids, host(w), ne)  # grouped with the device's own weights: bit for bit
        for name, a, b in zip(["table", "tok", "tok_off", "hit_row", "hit_w"], outs, want):
            assert np.array_equal(host(a)[: b.shape[0]].view(np.uint32), b.view(np.uint32)), (step, name)
    rec.graph.destroy()


def test_recorded_family_steps_replay_on_the_data_of_the_day(be, ora):
    """The q/k/v step with biases and the cache store, the sandwich norm and GeGLU inside one recording (three nodes,
    four with the separate v-bias launch of the storeless form): every replay works on what is in the buffers then,
    and equals the unrecorded calls bit for bit."""
    from allpaka_amd import synth as s

    rows, n_q, n_kv, hd, n = 5, 12, 2, 128, 2304
    g = s.rng(6, 1)
    qb, kb, vb = (dev(s.normal_f32(g, m * hd, 0.0, 0.5)) for m in (n_q, n_kv, n_kv))
    pg, gamma = dev(s.normal_f32(g, n, 1.0, 0.05)), dev(s.normal_f32(g, n, 1.0, 0.05))
    pos = torch.tensor([3, 0, 7, 1, 5], dtype=torch.int32, device="cuda")
    ropes = dev(ora.rope_table([3, 0, 7, 1, 5], ora.rope_inv_freq(hd, 1e6)))
    f16 = torch.float16
    q, k, v = (torch.zeros((rows, m * hd), dtype=f16, device="cuda") for m in (n_q, n_kv, n_kv))
    x, d, h = (torch.zeros((rows, n), dtype=f16, device="cuda") for _ in range(3))
    gate, up = torch.zeros(4000, dtype=f16, device="cuda"), torch.zeros(4000, dtype=f16, device="cuda")
    kc = torch.zeros((8, n_kv * hd), dtype=f16, device="cuda")
    vc = torch.zeros_like(kc)

    def step():
        be.attn_prologue_rows(q, k, v, n_q, n_kv, hd, 1e-6, ropes, q_bias=qb, k_bias=kb, v_bias=vb, cache_pos=pos, k_cache=kc, v_cache=vc)
        be.postnorm_add_rmsnorm_rows(x, d, pg, h, gamma, 1e-6)
        be.geglu_tanh(gate, up)

    with be.record() as rec:
        step()
    assert rec.graph.nodes == 3
    bufs = (q, k, v, x, d, gate, up)
    for it in range(3):
        gen = torch.Generator(device="cuda").manual_seed(50 + it)
        fresh = [torch.randn(b.shape, generator=gen, device="cuda").to(f16) for b in bufs]
        for b, f in zip(bufs, fresh):
            b.copy_(f)
        for t in (kc, vc, h):
            t.zero_()
        be.swiglu(torch.ones(64, device="cuda"), torch.ones(64, device="cuda"))  # unrecorded work in between
        rec.graph.launch()
        be.sync()
        got = [t.clone() for t in (q, k, v, x, h, gate, kc, vc)]
        for b, f in zip(bufs, fresh):
            b.copy_(f)
        for t in (kc, vc, h):
            t.zero_()
        step()
        be.sync()
        for name, a, b in zip("q k v x h gate kc vc".split(), got, (q, k, v, x, h, gate, kc, vc)):
            assert torch.equal(a, b), (it, name)
        assert be.take_faults() == 0
    rec.graph.destroy()

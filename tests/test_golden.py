"""The frozen fixtures of tests/golden/vectors.npz (written by tests/golden/make_golden.py).

CPU: the oracle still returns exactly what was frozen (same C source, same libm: bit for bit).
GPU: every op through the C ABI against the frozen outputs, to the bars of the parity tests.
"""
import os

import numpy as np
import pytest

from util import close_idiom, f16_ulp_diff, rel_err_f32

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz")
FORMATS = ["Q4K", "Q5K", "Q6K", "Q8_0", "Q2K", "Q3K", "Q5_0", "F16", "F32", "BF16"]
QK_TAGS = ["neox128", "neox64", "partial", "norm96"]


@pytest.fixture(scope="module")
def gold():
    with np.load(GOLDEN, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def same(a, b):
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8))


# ----------------------------------------------------------------------- CPU
def test_fixture_file_is_complete(gold):
    assert len(gold) == 156
    for name in FORMATS:
        assert f"embed.{name}.f16" in gold
    assert gold["moe.ids"].shape == (40, 8) and gold["argmax.pick"].shape == (5,)


def test_oracle_reproduces_the_frozen_outputs(gold, ora):
    g = gold
    for name in FORMATS:
        fmt = ora.FMT[name]
        t = g[f"embed.{name}.table"]
        assert same(ora.embed_rows(t, fmt, 5, 256, g["embed.ids"]), g[f"embed.{name}.f32"]), name
        assert same(ora.embed_rows(t, fmt, 5, 256, g["embed.ids"], out_f16=True), g[f"embed.{name}.f16"]), name
        assert same(ora.embed_rows(t, fmt, 5, 256, g["embed.ids"], scale=1.5), g[f"embed.{name}.f32.scaled"]), name
    for tag in ("a", "b", "ragged"):
        x, d, gamma = g[f"addnorm.{tag}.x"], g[f"addnorm.{tag}.d"], g[f"addnorm.{tag}.gamma"]
        wx, wh = x.copy(), np.zeros_like(x)
        ora.add_rmsnorm_rows(wx, d, wh, gamma, 1e-6)
        assert same(wx, g[f"addnorm.{tag}.f32.x"]) and same(wh, g[f"addnorm.{tag}.f32.h"]), tag
    for tag in QK_TAGS:
        rows, nq, nkv, hd, rot, style = (int(v) for v in g[f"qk.{tag}.meta"])
        ropes = ora.rope_table([int(p) for p in g[f"qk.{tag}.pos"]], ora.rope_inv_freq(rot, 1e6))
        assert same(ropes, g[f"qk.{tag}.ropes"]), tag
        wq, wk = g[f"qk.{tag}.q"].copy(), g[f"qk.{tag}.k"].copy()
        ora.qknorm_rope_rows(wq, wk, nq, nkv, hd, g[f"qk.{tag}.qw"], g[f"qk.{tag}.kw"], ropes, 1e-6, style=style)
        assert same(wq, g[f"qk.{tag}.f32.q"]) and same(wk, g[f"qk.{tag}.f32.k"]), tag
    w = g["swiglu.gate"].copy()
    ora.swiglu(w, g["swiglu.up"])
    assert same(w, g["swiglu.f32"])
    ids, wts = ora.route_rows(g["moe.logits"], 8, ora.SOFTMAX, True, 1.0, threads=2)
    assert same(ids, g["moe.ids"]) and same(wts, g["moe.w"])
    assert list(ids[7][:2]) == [5, 9]  # the tie: lower index first
    for got, name in zip(ora.moe_group(ids, wts, 128), ["table", "tok", "tok_off", "hit_row", "hit_w"]):
        assert same(got, g[f"moe.{name}"]), name
    wx, wh = g["moe.x"].copy(), np.zeros_like(g["moe.x"])
    ora.moe_combine_add_rmsnorm(wx, g["moe.flat"], g["moe.tok_off"], g["moe.hit_row"], g["moe.hit_w"], wh, g["moe.gamma"], 1e-6)
    assert same(wx, g["moe.combine.x"]) and same(wh, g["moe.combine.h"])
    assert same(np.array([ora.argmax_last(r) for r in g["argmax.logits"]], np.uint32), g["argmax.pick"])
    assert list(g["argmax.pick"][[1, 3]]) == [500, 599]  # ties: the last maximum
    w = g["geglu.gate"].copy()
    ora.geglu_tanh(w, g["geglu.up"])
    assert same(w, g["geglu.f32"])
    f16 = lambda a: a.astype(np.float16).view(np.uint16)  # noqa: E731
    for tag, conv in (("f32", lambda a: a.copy()), ("f16", f16)):
        xx, dd = conv(g["postnorm.x"]), conv(g["postnorm.d"])
        nd = np.zeros_like(dd)
        ora.add_rmsnorm_rows(dd.copy(), None, nd, g["postnorm.pg"], 1e-6)
        wx, wh = xx.copy(), np.zeros_like(xx)
        ora.add_rmsnorm_rows(wx, nd, wh, g["postnorm.gamma"], 1e-6)
        assert same(wx, g[f"postnorm.{tag}.x"]) and same(wh, g[f"postnorm.{tag}.h"]), tag
        wq, wk = conv(g["bias.q"]), conv(g["bias.k"])
        ora.qknorm_rope_rows(wq, wk, 28, 4, 128, None, None, g["bias.ropes"], 1e-6, q_bias=g["bias.qb"], k_bias=g["bias.kb"])
        assert same(wq, g[f"bias.{tag}.q"]) and same(wk, g[f"bias.{tag}.k"]), tag
    to, hr, hw = ora.moe_shared_hits(g["moe.tok_off"], g["moe.hit_row"], g["moe.hit_w"], 320)
    assert same(to, g["moe.shared.tok_off"]) and same(hr, g["moe.shared.hit_row"]) and same(hw, g["moe.shared.hit_w"])


# ----------------------------------------------------------------------- GPU
torch = None


@pytest.fixture(scope="module")
def be():
    global torch
    torch = pytest.importorskip("torch")
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


@pytest.mark.gpu
def test_device_embedding_equals_the_frozen_rows(gold, be, ora):
    import allpaka_amd as apk

    g = gold
    for name in FORMATS:
        qm = apk.QuantMat(be, dev(g[f"embed.{name}.table"]), ora.FMT[name], 5, 256)
        for key, dt, scale in ((f"embed.{name}.f32", torch.float32, 1.0), (f"embed.{name}.f16", torch.float16, 1.0),
                               (f"embed.{name}.f32.scaled", torch.float32, 1.5)):
            out = torch.zeros((4, 256), dtype=dt, device="cuda")
            qm.rows_into(dev(g["embed.ids"]), out, embed_scale=scale)
            assert same(host(out), g[key]), key


@pytest.mark.gpu
def test_device_layer_ops_match_the_frozen_outputs(gold, be, ora):
    g = gold
    f16 = lambda a: a.astype(np.float16).view(np.uint16)  # noqa: E731
    for tag in ("a", "b", "ragged"):
        x, d, gamma = g[f"addnorm.{tag}.x"], g[f"addnorm.{tag}.d"], g[f"addnorm.{tag}.gamma"]
        tx, th = dev(x), torch.zeros_like(dev(x))
        be.add_rmsnorm_rows(tx, dev(d), th, dev(gamma), 1e-6)
        assert same(host(tx), g[f"addnorm.{tag}.f32.x"])
        assert rel_err_f32(host(th), g[f"addnorm.{tag}.f32.h"]) <= 1e-5 and close_idiom(host(th), g[f"addnorm.{tag}.f32.h"])
        if f"addnorm.{tag}.f16.h" in g:
            tx, th = dev(f16(x)), torch.zeros_like(dev(f16(x)))
            be.add_rmsnorm_rows(tx, dev(f16(d)), th, dev(gamma), 1e-6)
            assert same(host(tx), g[f"addnorm.{tag}.f16.x"])
            assert f16_ulp_diff(host(th), g[f"addnorm.{tag}.f16.h"]) <= 2
    for tag in QK_TAGS:
        rows, nq, nkv, hd, rot, style = (int(v) for v in g[f"qk.{tag}.meta"])
        fn = be.qknorm_rope_norm if style else be.qknorm_rope_neox
        ropes, qw, kw = dev(g[f"qk.{tag}.ropes"]), dev(g[f"qk.{tag}.qw"]), dev(g[f"qk.{tag}.kw"])
        tq, tk = dev(g[f"qk.{tag}.q"]), dev(g[f"qk.{tag}.k"])
        fn(tq, tk, qw, kw, ropes, nq, nkv, hd, 1e-6, rot_dim=rot)
        for got, key in ((tq, f"qk.{tag}.f32.q"), (tk, f"qk.{tag}.f32.k")):
            assert rel_err_f32(host(got), g[key]) <= 1e-5 and close_idiom(host(got), g[key]), key
        tq, tk = dev(f16(g[f"qk.{tag}.q"])), dev(f16(g[f"qk.{tag}.k"]))
        fn(tq, tk, qw, kw, ropes, nq, nkv, hd, 1e-6, rot_dim=rot)
        assert same(host(tq), g[f"qk.{tag}.f16.q"]) and same(host(tk), g[f"qk.{tag}.f16.k"]), tag  # the definition, bit for bit
        # the rotary rows built on the device from the positions
        table = be.rope_table(dev(g[f"qk.{tag}.pos"]), dev(ora.rope_inv_freq(rot, 1e6)))
        assert np.max(np.abs(host(table) - g[f"qk.{tag}.ropes"])) <= 1.2e-7
    tg = dev(g["swiglu.gate"])
    be.swiglu(tg, dev(g["swiglu.up"]))
    assert rel_err_f32(host(tg), g["swiglu.f32"]) <= 1e-5 and close_idiom(host(tg), g["swiglu.f32"])
    tg = dev(f16(g["swiglu.gate"]))
    be.swiglu(tg, dev(f16(g["swiglu.up"])))
    assert f16_ulp_diff(host(tg), g["swiglu.f16"]) <= 2


@pytest.mark.gpu
def test_device_moe_chain_and_argmax_match_the_frozen_outputs(gold, be):
    g = gold
    ids, w = be.route_rows(dev(g["moe.logits"]), 8)
    assert same(host(ids), g["moe.ids"])
    assert np.array_equal(host(w), g["moe.w"])
    got = be.moe_permute(dev(g["moe.ids"]), dev(g["moe.w"]), 128)
    for a, name in zip(got, ["table", "tok", "tok_off", "hit_row", "hit_w"]):
        assert same(host(a), g[f"moe.{name}"]), name
    tx, th = dev(g["moe.x"]), torch.zeros_like(dev(g["moe.x"]))
    be.moe_combine_add_rmsnorm(tx, dev(g["moe.flat"]), got[2], got[3], got[4], th, dev(g["moe.gamma"]), 1e-6)
    assert same(host(tx), g["moe.combine.x"])
    assert rel_err_f32(host(th), g["moe.combine.h"]) <= 1e-5
    assert same(host(be.argmax_rows(dev(g["argmax.logits"]))), g["argmax.pick"])


@pytest.mark.gpu
def test_device_gemma_and_bias_steps_match_the_frozen_outputs(gold, be):
    g = gold
    f16 = lambda a: a.astype(np.float16).view(np.uint16)  # noqa: E731
    tg = dev(g["geglu.gate"])
    be.geglu_tanh(tg, dev(g["geglu.up"]))
    assert close_idiom(host(tg), g["geglu.f32"])
    for tag, conv in (("f32", lambda a: a), ("f16", f16)):
        tx, th = dev(conv(g["postnorm.x"])), torch.zeros_like(dev(conv(g["postnorm.x"])))
        be.postnorm_add_rmsnorm_rows(tx, dev(conv(g["postnorm.d"])), dev(g["postnorm.pg"]), th, dev(g["postnorm.gamma"]), 1e-6)
        if tag == "f16":
            assert same(host(tx), g["postnorm.f16.x"])
            assert f16_ulp_diff(host(th), g["postnorm.f16.h"]) <= 2
        else:
            for got, key in ((tx, "postnorm.f32.x"), (th, "postnorm.f32.h")):
                assert rel_err_f32(host(got), g[key]) <= 1e-5 and close_idiom(host(got), g[key]), key
        tq, tk, tv = dev(conv(g["bias.q"])), dev(conv(g["bias.k"])), dev(conv(g["bias.v"]))
        kc = torch.zeros((12, 4 * 128), dtype=torch.float16, device="cuda")
        vc = torch.zeros_like(kc)
        be.attn_prologue_rows(tq, tk, tv, 28, 4, 128, 1e-6, dev(g["bias.ropes"]), q_bias=dev(g["bias.qb"]), k_bias=dev(g["bias.kb"]),
                              v_bias=dev(g["bias.vb"]), cache_pos=dev(g["bias.pos"]), k_cache=kc, v_cache=vc)
        if tag == "f32":  # one add, then the reference's four products and two sums: bit for bit
            assert same(host(tq), g["bias.f32.q"]) and same(host(tk), g["bias.f32.k"])
        else:
            assert f16_ulp_diff(host(tq), g["bias.f16.q"]) <= 2 and f16_ulp_diff(host(tk), g["bias.f16.k"]) <= 2
        assert same(host(tv), g[f"bias.{tag}.v"]) and same(host(vc), g[f"bias.{tag}.vc"])
        assert f16_ulp_diff(host(kc), g[f"bias.{tag}.kc"]) <= (2 if tag == "f16" else 1)
    got = be.moe_shared_hits(dev(g["moe.tok_off"]), dev(g["moe.hit_row"]), dev(g["moe.hit_w"]), 320)
    for a, name in zip(got, ["tok_off", "hit_row", "hit_w"]):
        assert same(host(a), g[f"moe.shared.{name}"]), name

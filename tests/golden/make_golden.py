#!/usr/bin/env python3
"""Writes tests/golden/vectors.npz: small seeded inputs for every op together with the CPU oracle's
outputs, frozen.  The oracle itself is pinned by the reference's known-answer vectors
(tests/test_oracle_known_answers.py); these fixtures freeze what it returns on richer inputs, so that

  * a change of the oracle (or of the libm under it) that moves any output shows up on the CPU, and
  * the GPU path is also checked against files, not only against the oracle of the day.

Run from the repository root:  python tests/golden/make_golden.py
Everything here comes from this repository's own generators and oracle; nothing is read from the
reference at run time.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle as ora  # noqa: E402
from allpaka_amd import synth as s  # noqa: E402

FORMATS = ["Q4K", "Q5K", "Q6K", "Q8_0", "Q2K", "Q3K", "Q5_0", "F16", "F32", "BF16"]
SCALE_OFFS = {"Q8_0": (34, [0]), "Q2K": (84, [80, 82]), "Q3K": (110, [108]), "Q4K": (144, [0, 2]), "Q5K": (176, [0, 2]),
              "Q6K": (210, [208]), "Q5_0": (22, [0])}


def build():
    out = {}
    g = np.random.default_rng(20240607)

    def f16(a):
        return s.to_f16_bits(a)

    # embedding: every format, vocab 5, hidden 256, ids with a repeat
    ids = np.array([3, 0, 4, 3], np.uint32)
    out["embed.ids"] = ids
    for name in FORMATS:
        fmt = ora.FMT[name]
        rb = ora.expected_bytes(fmt, 256)
        raw = g.integers(0, 256, size=5 * rb, dtype=np.uint8)
        if name in SCALE_OFFS:
            bb, offs = SCALE_OFFS[name]
            blocks = raw.reshape(-1, bb)
            for o in offs:
                blocks[:, o + 1] &= 0x3B
        elif name == "F32":
            raw = s.normal_f32(g, 5 * 256).view(np.uint8).copy()
        else:
            raw.view(np.uint16)[:] &= np.uint16(0xBFFF)
        out[f"embed.{name}.table"] = raw
        out[f"embed.{name}.f32"] = ora.embed_rows(raw, fmt, 5, 256, ids)
        out[f"embed.{name}.f16"] = ora.embed_rows(raw, fmt, 5, 256, ids, out_f16=True)
        out[f"embed.{name}.f32.scaled"] = ora.embed_rows(raw, fmt, 5, 256, ids, scale=1.5)

    # residual add + RMSNorm
    for tag, rows, n in (("a", 2, 1024), ("b", 1, 5120), ("ragged", 2, 37)):
        x, d = s.normal_f32(g, (rows, n)), s.normal_f32(g, (rows, n))
        gamma = s.normal_f32(g, n, 1.0, 0.05)
        out[f"addnorm.{tag}.x"], out[f"addnorm.{tag}.d"], out[f"addnorm.{tag}.gamma"] = x, d, gamma
        wx, wh = x.copy(), np.zeros_like(x)
        ora.add_rmsnorm_rows(wx, d, wh, gamma, 1e-6)
        out[f"addnorm.{tag}.f32.x"], out[f"addnorm.{tag}.f32.h"] = wx, wh
        if n % 8 == 0:
            x16, d16 = f16(x), f16(d)
            wx, wh = x16.copy(), np.zeros_like(x16)
            ora.add_rmsnorm_rows(wx, d16, wh, gamma, 1e-6)
            out[f"addnorm.{tag}.f16.x"], out[f"addnorm.{tag}.f16.h"] = wx, wh

    # per-head QK-norm + RoPE: tiled geometry, partial rotary, adjacent-pair style
    for tag, rows, nq, nkv, hd, rot, style in (("neox128", 2, 4, 2, 128, 128, 0), ("neox64", 2, 3, 1, 64, 64, 0),
                                               ("partial", 2, 2, 1, 128, 64, 0), ("norm96", 2, 2, 2, 96, 96, 1)):
        q, k = s.normal_f32(g, (rows, nq * hd)), s.normal_f32(g, (rows, nkv * hd))
        qw, kw = s.normal_f32(g, hd, 1.0, 0.05), s.normal_f32(g, hd, 1.0, 0.05)
        pos = g.integers(0, 32768, size=rows).astype(np.uint32)
        ropes = ora.rope_table([int(p) for p in pos], ora.rope_inv_freq(rot, 1e6))
        meta = np.array([rows, nq, nkv, hd, rot, style], np.int64)
        out[f"qk.{tag}.meta"], out[f"qk.{tag}.q"], out[f"qk.{tag}.k"] = meta, q, k
        out[f"qk.{tag}.qw"], out[f"qk.{tag}.kw"], out[f"qk.{tag}.pos"], out[f"qk.{tag}.ropes"] = qw, kw, pos, ropes
        wq, wk = q.copy(), k.copy()
        ora.qknorm_rope_rows(wq, wk, nq, nkv, hd, qw, kw, ropes, 1e-6, style=style)
        out[f"qk.{tag}.f32.q"], out[f"qk.{tag}.f32.k"] = wq, wk
        wq, wk = f16(q), f16(k)
        ora.qknorm_rope_rows(wq, wk, nq, nkv, hd, qw, kw, ropes, 1e-6, style=style)
        out[f"qk.{tag}.f16.q"], out[f"qk.{tag}.f16.k"] = wq, wk

    # SwiGLU
    gate, up = s.normal_f32(g, 3001, 0.0, 3.0), s.normal_f32(g, 3001)
    out["swiglu.gate"], out["swiglu.up"] = gate, up
    w = gate.copy()
    ora.swiglu(w, up)
    out["swiglu.f32"] = w
    w = f16(gate)
    ora.swiglu(w, f16(up))
    out["swiglu.f16"] = w

    # router, grouping, combine
    logits = s.normal_f32(g, (40, 128))
    logits[7, [5, 9]] = 4.0  # an exact tie at the top: the lower index first
    out["moe.logits"] = logits
    ids_r, w_r = ora.route_rows(logits, 8, ora.SOFTMAX, True, 1.0, threads=2)
    out["moe.ids"], out["moe.w"] = ids_r, w_r
    table, tok, tok_off, hit_row, hit_w = ora.moe_group(ids_r, w_r, 128)
    out["moe.table"], out["moe.tok"], out["moe.tok_off"], out["moe.hit_row"], out["moe.hit_w"] = table, tok, tok_off, hit_row, hit_w
    flat, x = s.normal_f32(g, (40 * 8, 64)), s.normal_f32(g, (40, 64))
    gamma = s.normal_f32(g, 64, 1.0, 0.05)
    out["moe.flat"], out["moe.x"], out["moe.gamma"] = flat, x, gamma
    wx, wh = x.copy(), np.zeros_like(x)
    ora.moe_combine_add_rmsnorm(wx, flat, tok_off, hit_row, hit_w, wh, gamma, 1e-6)
    out["moe.combine.x"], out["moe.combine.h"] = wx, wh

    # greedy argmax (last maximum) with ties
    lg = s.normal_f32(g, (5, 600))
    lg[1, [10, 500, 333]] = 9.0
    lg[3, :] = 0.0
    out["argmax.logits"] = lg
    out["argmax.pick"] = np.array([ora.argmax_last(r) for r in lg], np.uint32)

    # (added after the arrays above: the generator's stream up to here, and with it every array above, is unchanged)
    # GeGLU with the tanh GELU
    gate, up = s.normal_f32(g, 2003, 0.0, 2.5), s.normal_f32(g, 2003)
    out["geglu.gate"], out["geglu.up"] = gate, up
    w = gate.copy()
    ora.geglu_tanh(w, up)
    out["geglu.f32"] = w
    w = f16(gate)
    ora.geglu_tanh(w, f16(up))
    out["geglu.f16"] = w

    # sandwich norm + next norm: x += rmsnorm(delta) * post_gamma; h = rmsnorm(x) * gamma
    x, d = s.normal_f32(g, (3, 2304)), s.normal_f32(g, (3, 2304), 0.0, 3.0)
    pg, gamma = s.normal_f32(g, 2304, 1.0, 0.05), s.normal_f32(g, 2304, 1.0, 0.05)
    out["postnorm.x"], out["postnorm.d"], out["postnorm.pg"], out["postnorm.gamma"] = x, d, pg, gamma
    for tag, xx, dd in (("f32", x, d), ("f16", f16(x), f16(d))):
        nd = np.zeros_like(dd)
        ora.add_rmsnorm_rows(dd.copy(), None, nd, pg, 1e-6)
        wx, wh = xx.copy(), np.zeros_like(xx)
        ora.add_rmsnorm_rows(wx, nd, wh, gamma, 1e-6)
        out[f"postnorm.{tag}.x"], out[f"postnorm.{tag}.h"] = wx, wh

    # q/k/v biases, no QK-norm, NeoX rotation, K/V cache store (28 + 4 heads of 128, three rows)
    rows, nq, nkv, hd = 3, 28, 4, 128
    q, k, v = s.normal_f32(g, (rows, nq * hd)), s.normal_f32(g, (rows, nkv * hd)), s.normal_f32(g, (rows, nkv * hd))
    qb, kb, vb = s.normal_f32(g, nq * hd, 0.0, 0.5), s.normal_f32(g, nkv * hd, 0.0, 0.5), s.normal_f32(g, nkv * hd, 0.0, 0.5)
    pos = np.array([5, 0, 9], np.uint32)
    ropes = ora.rope_table([int(p) for p in pos], ora.rope_inv_freq(hd, 1e6))
    out["bias.q"], out["bias.k"], out["bias.v"], out["bias.qb"], out["bias.kb"], out["bias.vb"] = q, k, v, qb, kb, vb
    out["bias.pos"], out["bias.ropes"] = pos, ropes
    for tag, conv, back in (("f32", lambda a: a.copy(), lambda a: a), ("f16", f16, None)):
        wq, wk = conv(q), conv(k)
        ora.qknorm_rope_rows(wq, wk, nq, nkv, hd, None, None, ropes, 1e-6, q_bias=qb, k_bias=kb)
        if tag == "f32":
            wv = v.copy()
            ora.add_bias_rows(wv, vb)
        else:
            wv = ora.f16_bits_to_f32(f16(v))
            ora.add_bias_rows(wv, vb)
            wv = ora.f32_to_f16_bits(wv)
        kc, vc = np.zeros((12, nkv * hd), np.uint16), np.zeros((12, nkv * hd), np.uint16)
        ora.kv_store_rows(wk, wv, pos, kc, vc)
        out[f"bias.{tag}.q"], out[f"bias.{tag}.k"], out[f"bias.{tag}.v"] = wq, wk, wv
        out[f"bias.{tag}.kc"], out[f"bias.{tag}.vc"] = kc, vc

    # the shared expert's hit in the lists of the grouping above
    to, hr, hw = ora.moe_shared_hits(tok_off, hit_row, hit_w, 40 * 8)
    out["moe.shared.tok_off"], out["moe.shared.hit_row"], out["moe.shared.hit_w"] = to, hr, hw
    return out


if __name__ == "__main__":
    data = build()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")
    np.savez_compressed(path, **data)
    print(f"{path}: {len(data)} arrays, {os.path.getsize(path) / 1024:.0f} KiB")

#!/usr/bin/env python3
"""Benchmark of the fused per-layer ops on ONE MI355X.

A "step" is one decoder layer's worth of the hot path at Qwen3-32B shapes,
T=2048 prefill rows, fp16 activations (the headline configuration):
    add+RMSNorm (attention norm) -> per-head QK-norm + NeoX RoPE ->
    add+RMSNorm (FFN norm) -> SwiGLU
i.e. 4 launches per layer, inputs resident in HBM.  Every op cycles through its
own pool of distinct buffer sets of more than 640 MB, so no launch is served
from the 256 MB last-level cache ("cold" = HBM numbers).  Every op is also
timed on its own, at every shape of the five benchmark configurations, with HIP events on the library's
stream (3 untimed launches first).  The JSON line carries
    value     = microseconds per layer (lower is better),
    roofline  = the dominant kernel (SwiGLU, 300 MiB per launch) against 8 TB/s,
    per_op    = us / GB/s / fraction of peak / launches for every op and shape,
    cpu_baseline = the CPU oracle (a C restatement of the reference's CPU path with
                   the reference's threading rules) timed on this box's host cores.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_GBS = 8000.0  # MI355X HBM3E peak
COLD_BYTES = 640e6  # every op rotates through at least this many distinct bytes

# HBM traffic of the dominant kernel per launch (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, KiB per dispatch, scaled by
# the same counters on apk_copy of a known size): read from the committed summary of those runs, so that the figure
# travels with the profile it came from; None when the summary has no row for the kernel.
TRAFFIC_PROFILE = os.path.join("profiles", "layer-ops_qwen3-32b_T2048_f16_hbm-traffic.md")


def traffic_from_profile(kernel):
    import re

    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
    except OSError:
        return None
    m = re.search(r"^\| " + re.escape(kernel) + r" \| \d+ \| \d+ \| (\d+) \|", text, re.M)
    return int(m.group(1)) if m else None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=60)
    ap.add_argument("--warmup", type=int, default=12)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--rows", type=int, default=2048, help="prefill rows T of the timed step")
    ap.add_argument("--shapes", choices=["all", "headline"], default="all",
                    help="headline: only the timed layer chain and its per-op timings (what the rocprof summaries are made from)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path is row-parallel and shards by rows with no "
              f"communication); --gpus {args.gpus} is not run", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import allpaka_amd.lib as apklib
    from allpaka_amd import synth

    L = apklib.load()  # raises if libapk_hip.so is not built: no fallback
    h = C.c_void_p()
    apklib.check(L.apk_init(0, C.byref(h)))
    dev = torch.device("cuda", 0)
    F16, F32 = apklib.F16, apklib.F32
    gen = torch.Generator(device=dev).manual_seed(0xA11A)

    def randn(shape, dtype=torch.float16):
        return torch.randn(shape, generator=gen, device=dev, dtype=torch.float32).to(dtype)

    def pool(set_bytes, make):
        """enough distinct sets that one cycle touches more than COLD_BYTES"""
        return [make() for _ in range(max(3, int(COLD_BYTES // set_bytes) + 1))]

    def p(t):
        return t.data_ptr()

    def sync():
        apklib.check(L.apk_sync(h))

    # ~2 ms of plain copies: what runs between a restore of inputs (which ends in a wait, so the GPU goes idle and its
    # clocks drop) and the launches that are timed, so that every timed batch starts on a GPU in its streaming state
    warm_half = 96 << 20  # (not the 100 MiB of the calibration copy below: a profile tells the two launch sizes apart)
    warm_buf = torch.empty(2 * warm_half, dtype=torch.uint8, device=dev)
    warm_buf.view(torch.float32).normal_()

    def busy(n=64):
        for _ in range(n):
            apklib.check(L.apk_copy(h, p(warm_buf), p(warm_buf) + warm_half, warm_half))

    def timed(fn, reps, batches=3, refresh=None, span=None):
        """microseconds per call of fn(i): HIP events on the library's stream around back-to-back launches, after
        3 untimed calls; the median over the timed batches.  refresh: called (untimed, then waited for) ahead of the
        warm-up and of every batch -- ops that work in place on data that would decay (SwiGLU: gate <- silu(gate) * up
        applied again and again runs towards zeros and subnormals, which stream 3-4 % faster than activations) get their
        inputs back there; span: the longest batch the op's pool allows between two refreshes (a batch is cut to it and
        the number of batches grows so that about `reps * batches` launches are still timed)."""
        if span is not None and reps > span - 3:  # three sets of the pool are left to the untimed launches of a batch
            batches = -(-reps * batches // (span - 3))
            reps = span - 3

        def fresh():
            if refresh is not None:
                sync()
                refresh()
                torch.cuda.synchronize()
                busy()

        if refresh is None:
            for i in range(3):
                fn(i)
        ms = C.c_float()
        avgs = []
        for bi in range(batches):
            if refresh is not None:
                # restored inputs, then three untimed launches on sets the timed ones do not touch, so that a batch
                # does not start on an idle GPU (the wait that ends the restore lets it go idle)
                fresh()
                for i in range(3):
                    fn(reps + i)
            apklib.check(L.apk_timer_begin(h))
            for i in range(reps):
                fn(i if refresh is not None else bi * reps + i)
            apklib.check(L.apk_timer_end(h, C.byref(ms)))
            avgs.append(ms.value * 1000.0 / reps)
        return sorted(avgs)[len(avgs) // 2]

    per_op = []

    def record(op, shape, us, nbytes, launches=1, note=None):
        gbs = nbytes / us / 1e3
        e = {"op": op, "shape": shape, "us": round(us, 3), "bytes": int(nbytes), "GBps": round(gbs, 1),
             "frac_of_peak": round(gbs / PEAK_GBS, 4), "launches": launches}
        if note:
            e["note"] = note
        per_op.append(e)
        return e

    # ------------------------------------------------ Qwen3-32B, fp16 (configs 2, 3)
    m = synth.MODELS["qwen3-32b"]
    H, NQ, NKV, HD, FF, EPS = m["hidden"], m["n_q"], m["n_kv"], m["head_dim"], m["ffn"], m["eps"]
    T = args.rows
    b = 2
    # one seeded set of layer inputs (allpaka_amd/synth.py), the same values the CPU leg runs on; the device keeps
    # them as fp16 and every pool set below is a copy of it (the pools only defeat the last-level cache)
    lay = synth.layer_inputs("qwen3-32b", T)

    def up16(a):
        return torch.from_numpy(a).to(dev).half()

    src = {name: up16(lay[name]) for name in ("x", "delta", "q", "k", "gate", "up")}
    gamma1, gamma2 = torch.from_numpy(lay["gamma1"]).to(dev), torch.from_numpy(lay["gamma2"]).to(dev)
    qw, kw = torch.from_numpy(lay["qw"]).to(dev), torch.from_numpy(lay["kw"]).to(dev)
    inv = torch.tensor(np.float32(m["theta"]) ** (-2.0 * np.arange(HD // 2, dtype=np.float32) / np.float32(HD)), device=dev)
    pos = torch.arange(T, dtype=torch.int32, device=dev)
    rope = torch.empty((T, HD // 2, 2), dtype=torch.float32, device=dev)
    torch.cuda.synchronize()
    apklib.check(L.apk_rope_table(h, p(pos), p(inv), T, HD // 2, p(rope)))
    sync()
    an = pool(3 * T * H * b, lambda: dict(x=src["x"].clone(), d=src["delta"].clone(), h=torch.empty((T, H), dtype=torch.float16, device=dev)))
    qk = pool(T * (NQ + NKV) * HD * b, lambda: dict(q=src["q"].clone(), k=src["k"].clone()))
    # SwiGLU works in place (gate <- silu(gate) * up): applied to the same buffer again and again the gate decays to
    # zeros and subnormals, which stream faster than activations.  So its pool holds one set per step of the timed loop
    # (every launch there sees fresh activations; 210 MB a set), and the per-op timing below restores the gates from
    # the pristine copy between batches that are no longer than the pool.
    n_sw = max(6, int(COLD_BYTES // (2 * T * FF * b)) + 1, min(args.steps + args.warmup, 160))
    sw = [dict(gate=src["gate"].clone(), up=src["up"].clone()) for _ in range(n_sw)]
    gate0 = src["gate"]
    del src
    torch.cuda.synchronize()

    def restore_gates(sets, pristine):
        for s_ in sets:
            s_["gate"].copy_(pristine)

    def dead_fraction(sets):
        """fraction of gate elements that are zero, subnormal or not finite (outside every timed region)"""
        bad = tot = 0
        for s_ in sets:
            g_ = s_["gate"]
            tiny = torch.finfo(g_.dtype).tiny
            bad += int(((g_.abs() < tiny) | ~torch.isfinite(g_)).sum())
            tot += g_.numel()
        return bad / tot

    def op_addnorm(i, gamma=gamma1, rows=T):
        s = an[i % len(an)]
        apklib.check(L.apk_add_rmsnorm_rows(h, p(s["x"]), p(s["d"]), p(s["h"]), p(gamma), H, rows, EPS, F16))

    def op_qkrope(i, rows=T):
        s = qk[i % len(qk)]
        apklib.check(L.apk_qknorm_rope_neox(h, p(s["q"]), p(s["k"]), p(qw), p(kw), p(rope), rows, NQ, NKV, HD, HD, EPS, F16))

    def op_swiglu(i, rows=T):
        s = sw[i % len(sw)]
        apklib.check(L.apk_swiglu(h, p(s["gate"]), p(s["up"]), rows * FF, F16))

    def layer(i):
        op_addnorm(2 * i)
        op_qkrope(i)
        op_addnorm(2 * i + 1, gamma2)
        op_swiglu(i)

    # ------------------------------------------------------------ timed steps
    for i in range(args.warmup):
        layer(i)
    sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ms = C.c_float()
    apklib.check(L.apk_timer_begin(h))
    for i in range(args.steps):
        layer(i + args.warmup)
    apklib.check(L.apk_timer_end(h, C.byref(ms)))
    sync()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1000.0
    ms_per_step = wall_ms / args.steps
    us_layer_events = ms.value * 1000.0 / args.steps
    # the timed loop ran on live data: every SwiGLU launch of it (warm-up included) had a set of its own when the pool
    # is at least that long; otherwise some sets were gated more than once
    dead_chain = dead_fraction(sw)

    # ---------------------------------------------- per-op timings, headline shape
    reps = max(20, args.steps)
    tag = f"qwen3-32b T={T} f16"
    bytes_addnorm = 4 * T * H * b + 4 * H
    bytes_qkrope = 2 * T * (NQ + NKV) * HD * b + T * (HD // 2) * 8 + 2 * HD * 4
    bytes_swiglu = 3 * T * FF * b
    e_an = record("add_rmsnorm", tag, timed(op_addnorm, reps), bytes_addnorm)
    e_qk = record("qknorm_rope_neox", tag, timed(op_qkrope, reps), bytes_qkrope)
    dom = record("swiglu", tag, timed(op_swiglu, reps, refresh=lambda: restore_gates(sw, gate0), span=len(sw)), bytes_swiglu)
    dead_op = dead_fraction(sw)  # after the last batch: every set gated at most once since its refresh
    assert dead_op < 0.01, f"SwiGLU was timed on decayed gates: {dead_op:.4f} zero, subnormal or not finite"
    if n_sw >= args.steps + args.warmup:  # a set per step: the timed steps saw live gates too (a longer run than the pool
        assert dead_chain < 0.01, f"the timed steps ran on decayed gates: {dead_chain:.4f}"  # allows reuses sets; it is reported, not refused)
    # QK-norm + RoPE with the K/V cache store fused in (one launch; the cache planes of one layer, capacity T)
    kvp = [dict(v=randn((T, NKV * HD)), kc=torch.empty((T, NKV * HD), dtype=torch.float16, device=dev),
                vc=torch.empty((T, NKV * HD), dtype=torch.float16, device=dev)) for _ in range(len(qk))]
    torch.cuda.synchronize()
    bytes_qkkv = bytes_qkrope + T * NKV * HD * b + 2 * T * NKV * HD * 2 + T * 4
    us = timed(lambda i: apklib.check(L.apk_qknorm_rope_kv_store(
        h, p(qk[i % len(qk)]["q"]), p(qk[i % len(qk)]["k"]), p(kvp[i % len(qk)]["v"]), p(qw), p(kw), p(rope), p(pos),
        p(kvp[i % len(qk)]["kc"]), p(kvp[i % len(qk)]["vc"]), T, T, NQ, NKV, HD, HD, EPS, F16)), reps)
    e_kv = record("qknorm_rope_neox + K/V cache store (one launch)", tag, us, bytes_qkkv)
    cp_bytes = T * FF * b
    record("copy (plain stream)", f"{cp_bytes >> 20} MiB -> {cp_bytes >> 20} MiB",
           timed(lambda i: apklib.check(L.apk_copy(h, p(sw[i % len(sw)]["up"]), p(sw[i % len(sw)]["gate"]), cp_bytes)), reps), 2 * cp_bytes)
    sync()
    restore_gates(sw, gate0)
    torch.cuda.synchronize()

    # the kernels behind the headline ops, by the names the host launches them under (apk_plan_*: the same choice the
    # entries make for these sizes), for the record's roofline object
    def kernel_of(fn, *a):
        pl = apklib.Plan()
        apklib.check(fn(*a, C.byref(pl)))
        return pl.kernel.decode()

    headline_kernels = []
    for e_, kname in ((dom, "apk_swiglu_f16"),
                      (e_an, kernel_of(L.apk_plan_add_rmsnorm_rows, H, T, F16)),
                      (e_qk, kernel_of(L.apk_plan_qknorm_rope, T, NQ, NKV, HD, HD, 0, F16, 0)),
                      (e_kv, kernel_of(L.apk_plan_qknorm_rope, T, NQ, NKV, HD, HD, 0, F16, 1))):
        headline_kernels.append({"kernel": kname, "op": e_["op"], "us": e_["us"], "bytes": e_["bytes"], "GBps": e_["GBps"],
                                 "frac": e_["frac_of_peak"], "traffic": traffic_from_profile(kname)})

    # The practical ceiling at each op's size: a plain copy (one 16-byte tile per lane, out of place) moving
    # the same number of bytes.  Every launch pays a fixed ~2 us before it streams at ~6.8 TB/s, so a
    # ~76 MB op cannot reach the fraction of peak a 300 MB op does.
    cp_pool = torch.empty(int(COLD_BYTES * 1.1) // 4 * 4, dtype=torch.uint8, device=dev)
    cp_pool.view(torch.float32).normal_()  # not zeros: a stream of zeros runs 3-4 % faster than one of activations
    torch.cuda.synchronize()
    for name, nb in (("add_rmsnorm", bytes_addnorm), ("qknorm_rope_neox", bytes_qkrope), ("embed_rows Q4_K->f16", T * (2880 + 4 + H * 2))):
        half = nb // 2 // 4096 * 4096
        nset = cp_pool.numel() // (2 * half)
        us = timed(lambda i: apklib.check(L.apk_copy(h, p(cp_pool) + (i % nset) * 2 * half, p(cp_pool) + (i % nset) * 2 * half + half, half)), reps)
        record(f"copy (plain stream) of the bytes of {name}", f"{2 * half / 1e6:.1f} MB moved", us, 2 * half, note="ceiling at this size")
    del cp_pool

    if args.shapes == "all":
        # small-T shapes of the same model: launch-latency bound, reported as us/launch
        for rows, label in ((1, "decode T=1"), (6, "verify T=6"), (64, "batched decode, 64 rows with own positions")):
            sh = f"qwen3-32b {label} f16"
            record("add_rmsnorm", sh, timed(lambda i: op_addnorm(i, rows=rows), 200), 4 * rows * H * b + 4 * H, note="launch-bound")
            record("qknorm_rope_neox", sh, timed(lambda i: op_qkrope(i, rows=rows), 200),
                   2 * rows * (NQ + NKV) * HD * b + rows * (HD // 2) * 8 + 2 * HD * 4, note="launch-bound")
            record("swiglu", sh, timed(lambda i: op_swiglu(i, rows=rows), 200), 3 * rows * FF * b, note="launch-bound")
            us = timed(lambda i: apklib.check(L.apk_layer_prologue(
                h, p(an[i % len(an)]["x"]), p(an[i % len(an)]["d"]), p(an[i % len(an)]["h"]), p(gamma1), H,
                p(qk[i % len(qk)]["q"]), p(qk[i % len(qk)]["k"]), p(qw), p(kw), p(rope), rows, NQ, NKV, HD, HD, EPS, F16)), 200)
            record("layer_prologue (add_rmsnorm || qknorm_rope, one launch)", sh, us,
                   4 * rows * H * b + 4 * H + 2 * rows * (NQ + NKV) * HD * b + rows * (HD // 2) * 8 + 2 * HD * 4, note="launch-bound")
        # a decode step's QK-norm + RoPE + K/V cache store with the rotary angles taken from the device positions inside the
        # launch, against the table built by a launch of its own and then the table form (what a recorded decode chain
        # runs once per token and once per layer, respectively)
        for rows, label in ((1, "decode T=1"), (64, "batched decode, 64 rows with own positions")):
            sh = f"qwen3-32b {label} f16"
            nbp = 2 * rows * (NQ + NKV) * HD * b + rows * NKV * HD * b + 2 * rows * NKV * HD * 2 + rows * 4 + (HD // 2) * 4 + 2 * HD * 4
            us = timed(lambda i: apklib.check(L.apk_qknorm_rope_pos(
                h, p(qk[i % len(qk)]["q"]), p(qk[i % len(qk)]["k"]), p(kvp[i % len(qk)]["v"]), p(qw), p(kw), p(pos), p(inv),
                p(kvp[i % len(qk)]["kc"]), p(kvp[i % len(qk)]["vc"]), T, rows, NQ, NKV, HD, HD, 0, EPS, F16)), 200)
            record("qknorm_rope_pos: angles from positions in the launch + K/V cache store (one launch)", sh, us, nbp, note="launch-bound")

            def table_then_op(i, rows=rows):
                apklib.check(L.apk_rope_table(h, p(pos), p(inv), rows, HD // 2, p(rope)))
                apklib.check(L.apk_qknorm_rope_kv_store(
                    h, p(qk[i % len(qk)]["q"]), p(qk[i % len(qk)]["k"]), p(kvp[i % len(qk)]["v"]), p(qw), p(kw), p(rope), p(pos),
                    p(kvp[i % len(qk)]["kc"]), p(kvp[i % len(qk)]["vc"]), T, rows, NQ, NKV, HD, HD, EPS, F16))
            us = timed(table_then_op, 200)
            record("rope_table, then qknorm_rope + K/V cache store (two launches)", sh, us, nbp + rows * (HD // 2) * 16, launches=2, note="launch-bound")
        apklib.check(L.apk_rope_table(h, p(pos), p(inv), T, HD // 2, p(rope)))  # the full table again
        # the decode chain of a whole model (64 layers x 4 launches) issued op by op, and recorded once
        # and replayed with one submission; and the 3-launch form with the fused prologue
        NL = 64
        for rows, label in ((1, "decode T=1"), (6, "verify T=6"), (64, "batched decode, 64 rows")):
            sh = f"qwen3-32b {label} f16, {NL} layers"
            lb = 2 * (4 * rows * H * b + 4 * H) + 2 * rows * (NQ + NKV) * HD * b + rows * (HD // 2) * 8 + 2 * HD * 4 + 3 * rows * FF * b

            def chain4(j):
                for l in range(NL):
                    op_addnorm(2 * (j * NL + l), rows=rows)
                    op_qkrope(j * NL + l, rows=rows)
                    op_addnorm(2 * (j * NL + l) + 1, gamma2, rows=rows)
                    op_swiglu(j * NL + l, rows=rows)

            def chain3(j):
                for l in range(NL):
                    i = j * NL + l
                    apklib.check(L.apk_layer_prologue(
                        h, p(an[(2 * i) % len(an)]["x"]), p(an[(2 * i) % len(an)]["d"]), p(an[(2 * i) % len(an)]["h"]), p(gamma1), H,
                        p(qk[i % len(qk)]["q"]), p(qk[i % len(qk)]["k"]), p(qw), p(kw), p(rope), rows, NQ, NKV, HD, HD, EPS, F16))
                    op_addnorm(2 * i + 1, gamma2, rows=rows)
                    op_swiglu(i, rows=rows)

            for chain, nl, name in ((chain4, 4, "layer chain"), (chain3, 3, "layer chain with fused prologue")):
                us = timed(chain, 6) / NL
                record(f"{name}, op by op", sh, us, lb, launches=nl, note="launch-bound; us per layer")
                g = C.c_void_p()
                apklib.check(L.apk_capture_begin(h))
                chain(0)
                apklib.check(L.apk_capture_end(h, C.byref(g)))
                us = timed(lambda i: apklib.check(L.apk_graph_launch(h, g)), 12) / NL
                record(f"{name}, recorded once and replayed", sh, us, lb, launches=nl, note="launch-bound; us per layer")
                apklib.check(L.apk_graph_destroy(h, g))
        # the same rows with the adjacent-pair rotation and no QK-norm: the prologue of the Llama-family layouts
        # (32 q heads and 8 k heads of 128: the leading heads of the same buffers)
        lq, lkv = 32, 8
        us = timed(lambda i: apklib.check(L.apk_qknorm_rope_norm(h, p(qk[i % len(qk)]["q"]), p(qk[i % len(qk)]["k"]), None, None, p(rope),
                                                                 T, lq, lkv, HD, HD, EPS, F16)), reps)
        record("rope, adjacent pairs, no QK-norm", f"32 q + 8 k heads of 128, T={T} f16", us, 2 * T * (lq + lkv) * HD * b + T * HD * 4)
        # projection biases, the rotation and the K/V cache store as one call (28 q + 4 k heads of 128, biases on q, k, v,
        # no QK-norm: the geometry of the bias-carrying Qwen2.5-7B), on the leading heads of the same buffers
        bq, bkv = 28, 4
        qbias, kbias, vbias = randn((bq * HD,), torch.float32), randn((bkv * HD,), torch.float32), randn((bkv * HD,), torch.float32)
        pro = []
        for i in range(len(qk)):
            a = apklib.AttnPrologue()
            a.q, a.k, a.v = p(qk[i]["q"]), p(qk[i]["k"]), p(kvp[i]["v"])
            a.q_bias, a.k_bias, a.v_bias, a.rope = p(qbias), p(kbias), p(vbias), p(rope)
            a.cache_pos, a.k_cache, a.v_cache, a.capacity = p(pos), p(kvp[i]["kc"]), p(kvp[i]["vc"]), T
            a.rows, a.n_q, a.n_kv, a.head_dim, a.rot_dim, a.eps, a.dtype = T, bq, bkv, HD, HD, EPS, F16
            pro.append(a)
        us = timed(lambda i: apklib.check(L.apk_attn_prologue_rows(h, C.byref(pro[i % len(pro)]))), reps)
        record("attn_prologue: q/k/v biases + rope + K/V cache store (one launch)", f"28 q + 4 k heads of 128, T={T} f16", us,
               2 * T * (bq + 2 * bkv) * HD * b + 2 * T * bkv * HD * 2 + T * HD * 4 + T * 4 + (bq + 2 * bkv) * HD * 4)
        # what fusing the residual add into the norm buys: the same result as two launches of this library's own ops
        us = timed(lambda i: (apklib.check(L.apk_add_assign(h, p(an[i % len(an)]["x"]), p(an[i % len(an)]["d"]), T * H, F16)),
                              apklib.check(L.apk_add_rmsnorm_rows(h, p(an[i % len(an)]["x"]), None, p(an[i % len(an)]["h"]), p(gamma1), H, T, EPS, F16))), reps)
        record("UNFUSED residual add, then RMSNorm (two launches)", tag, us, 3 * T * H * b + 2 * T * H * b + 4 * H, launches=2,
               note="for comparison with add_rmsnorm")
        # the sandwich norm (x += rmsnorm(delta) * post_gamma) and the next norm as one launch: the bytes of add_rmsnorm
        us = timed(lambda i: apklib.check(L.apk_postnorm_add_rmsnorm_rows(h, p(an[i % len(an)]["x"]), p(an[i % len(an)]["d"]), p(gamma2),
                                                                          p(an[i % len(an)]["h"]), p(gamma1), H, T, EPS, F16)), reps)
        record("postnorm_add_rmsnorm (sandwich norm + next norm, one launch)", tag, us, bytes_addnorm + 4 * H)
        del an, qk, sw, kvp
        # the same headline shape with f32 activations, the reference's own activation type (f64 statistics,
        # the reference's operation order): twice the bytes per launch
        f32 = torch.float32
        an32 = pool(3 * T * H * 4, lambda: dict(x=randn((T, H), f32), d=randn((T, H), f32), h=torch.empty((T, H), dtype=f32, device=dev)))
        torch.cuda.synchronize()
        us = timed(lambda i: apklib.check(L.apk_add_rmsnorm_rows(h, p(an32[i % len(an32)]["x"]), p(an32[i % len(an32)]["d"]),
                                                                 p(an32[i % len(an32)]["h"]), p(gamma1), H, T, EPS, F32)), reps)
        record("add_rmsnorm", f"qwen3-32b T={T} f32", us, 4 * T * H * 4 + 4 * H)
        del an32
        qk32 = pool(T * (NQ + NKV) * HD * 4, lambda: dict(q=randn((T, NQ * HD), f32), k=randn((T, NKV * HD), f32)))
        torch.cuda.synchronize()
        us = timed(lambda i: apklib.check(L.apk_qknorm_rope_neox(h, p(qk32[i % len(qk32)]["q"]), p(qk32[i % len(qk32)]["k"]), p(qw), p(kw),
                                                                 p(rope), T, NQ, NKV, HD, HD, EPS, F32)), reps)
        record("qknorm_rope_neox", f"qwen3-32b T={T} f32", us, 2 * T * (NQ + NKV) * HD * 4 + T * (HD // 2) * 8 + 2 * HD * 4)
        del qk32
        gate32 = randn((T, FF), f32)
        sw32 = [dict(gate=gate32.clone(), up=randn((T, FF), f32)) for _ in range(8)]  # 419 MB a set
        torch.cuda.synchronize()
        us = timed(lambda i: apklib.check(L.apk_swiglu(h, p(sw32[i % len(sw32)]["gate"]), p(sw32[i % len(sw32)]["up"]), T * FF, F32)), reps,
                   refresh=lambda: restore_gates(sw32, gate32), span=len(sw32))
        assert dead_fraction(sw32) < 0.01
        record("swiglu", f"qwen3-32b T={T} f32", us, 3 * T * FF * 4)
        del sw32, gate32
        other_shapes(args, L, h, apklib, synth, torch, gen, dev, randn, pool, p, timed, record, reps, m, qw, kw, rope, restore_gates, dead_fraction, busy)
    sync()

    faults = C.c_uint32()
    apklib.check(L.apk_take_faults(h, C.byref(faults)))
    stats = [C.c_uint64() for _ in range(4)]
    L.apk_stats(h, *[C.byref(v) for v in stats])

    # ------------------------------------------------------------ cpu baseline
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(np, lay, T, H, NQ, NKV, HD, FF, EPS)

    layer_bytes = 2 * bytes_addnorm + bytes_qkrope + bytes_swiglu
    out = {
        "metric": "us/layer, fused layer ops (2x add+RMSNorm, QK-norm+RoPE, SwiGLU), Qwen3-32B shape",
        "value": round(us_layer_events, 3),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"configs[2]: Qwen3-32B fused layer ops, T={T} prefill rows, fp16 activations, "
                               f"hidden {H}, {NQ}q/{NKV}kv heads x {HD}, ffn {FF}; every op rotates through >= 640 MB of "
                               "distinct buffers so every launch streams from HBM",
                   "launches_per_layer": 4, "rows": T},
        "roofline": {"bound": "hbm", "kernel": "apk_swiglu_f16", "achieved": dom["GBps"], "peak": PEAK_GBS, "unit": "GB/s",
                     "frac": round(dom["GBps"] / PEAK_GBS, 4), "traffic": traffic_from_profile("apk_swiglu_f16"),
                     "traffic_source": TRAFFIC_PROFILE,
                     "algorithmic_bytes_per_launch": dom["bytes"], "avg_launch_us": dom["us"],
                     "gate_dead_fraction": {"after_timed_steps": round(dead_chain, 6), "after_per_op_timing": round(dead_op, 6),
                                            "sets": n_sw, "a_set_per_step": n_sw >= args.steps + args.warmup,
                                            "note": "share of SwiGLU gate elements that are zero, subnormal or not finite after the "
                                                    "run; the gates are restored from a pristine copy between timed batches"},
                     "kernels": headline_kernels},
        "layer_algorithmic_bytes": int(layer_bytes),
        "layer_GBps": round(layer_bytes / us_layer_events / 1e3, 1),
        "layer_frac_of_peak": round(layer_bytes / us_layer_events / 1e3 / PEAK_GBS, 4),
        "cpu_baseline": cpu,
        "per_op": per_op,
        "device_faults": faults.value,
        "stats": {"calls": stats[0].value, "dispatches": stats[1].value, "encode_ns": stats[2].value, "wait_ns": stats[3].value},
    }
    L.apk_shutdown(h)
    print(json.dumps(out))


def other_shapes(args, L, h, apklib, synth, torch, gen, dev, randn, pool, p, timed, record, reps, m, qw, kw, rope, restore_gates, dead_fraction, busy):
    """Embedding gathers, the Qwen3-0.6B f32 shapes and the MoE layer ops (inputs from a seeded device generator: these
    shapes have no CPU leg of their own in the timed step)."""
    F16, F32 = apklib.F16, apklib.F32
    H, HD, EPS, T = m["hidden"], m["head_dim"], m["eps"], args.rows
    check = apklib.check

    # embedding gather, Q4_K table [151936 x 5120] -> fp16 rows (config 2)
    vocab = m["vocab"]
    rb = L.apk_row_bytes(apklib.FMT_Q4K, H)
    table = torch.randint(0, 256, (vocab, H // 256, 144), generator=gen, device=dev, dtype=torch.uint8)
    dd = (torch.randn((vocab, H // 256, 2), generator=gen, device=dev).abs() * (0.02 / 63.0)).half()
    table[:, :, 0:4] = dd.view(torch.uint8).reshape(vocab, H // 256, 4)
    ids = torch.randint(0, vocab, (8, T), generator=gen, device=dev, dtype=torch.int32)
    outs = pool(T * H * 2, lambda: torch.empty((T, H), dtype=torch.float16, device=dev))
    torch.cuda.synchronize()
    for rows in (1, 6, T):
        us = timed(lambda i: check(L.apk_embed_rows(h, apklib.FMT_Q4K, p(table), vocab, H, p(ids[i % 8]), rows,
                                                    p(outs[i % len(outs)]), F16)), 200 if rows < T else reps)
        record("embed_rows Q4_K->f16", f"qwen3-32b T={rows}", us, rows * (rb + 4 + H * 2), note=None if rows == T else "launch-bound")
    del table
    # the same gather from the other common embedding formats of GGUF files (random bytes; the f16 scale
    # fields are whatever the bytes give -- the kernels do not care)
    for name, fmt in (("Q6_K", apklib.FMT_Q6K), ("Q8_0", apklib.FMT_Q8_0), ("Q5_K", apklib.FMT_Q5K)):
        rbx = L.apk_row_bytes(fmt, H)
        tb = torch.randint(0, 256, (vocab * rbx,), generator=gen, device=dev, dtype=torch.uint8)
        torch.cuda.synchronize()
        us = timed(lambda i: check(L.apk_embed_rows(h, fmt, p(tb), vocab, H, p(ids[i % 8]), T, p(outs[i % len(outs)]), F16)), reps)
        record(f"embed_rows {name}->f16", f"qwen3-32b T={T}", us, T * (rbx + 4 + H * 2))
        if name == "Q6_K":
            # a range of rows with no id list: a [8192 x 5120] slice of the same bytes widened to fp16, the step the
            # reference runs ahead of a dense GEMM on a quantized weight (the table rotates through 8192-row windows)
            wrows = 8192
            wouts = pool(wrows * H * 2, lambda: torch.empty((wrows, H), dtype=torch.float16, device=dev))
            us = timed(lambda i: check(L.apk_dequant_rows(h, fmt, p(tb), vocab, H, (i % 16) * wrows, wrows, p(wouts[i % len(wouts)]), F16)), reps)
            record("dequant_rows Q6_K->f16 (row range, no id list)", f"[{wrows} x {H}] weight", us, wrows * (rbx + H * 2))
            del wouts
        del tb
    del outs

    # Qwen3-0.6B shapes, f32 activations (configs 0 and 1)
    m0 = synth.MODELS["qwen3-0.6b"]
    H0, NQ0, NKV0, FF0, V0 = m0["hidden"], m0["n_q"], m0["n_kv"], m0["ffn"], m0["vocab"]
    T0 = 512
    f32 = torch.float32
    an0 = pool(3 * T0 * H0 * 4, lambda: dict(x=randn((T0, H0), f32), d=randn((T0, H0), f32), h=torch.empty((T0, H0), dtype=f32, device=dev)))
    qk0 = pool(T0 * (NQ0 + NKV0) * HD * 4, lambda: dict(q=randn((T0, NQ0 * HD), f32), k=randn((T0, NKV0 * HD), f32)))
    sw0 = pool(2 * T0 * FF0 * 4, lambda: dict(gate=randn((T0, FF0), f32), up=randn((T0, FF0), f32)))
    g0 = 1 + 0.05 * randn(H0, f32)
    q8 = torch.randint(0, 256, (V0, H0 // 32, 34), generator=gen, device=dev, dtype=torch.uint8)
    sc = (torch.randn((V0, H0 // 32, 1), generator=gen, device=dev).abs() * (0.02 / 127.0)).half()
    q8[:, :, 0:2] = sc.view(torch.uint8).reshape(V0, H0 // 32, 2)
    ids0 = torch.randint(0, V0, (8, T0), generator=gen, device=dev, dtype=torch.int32)
    torch.cuda.synchronize()
    for rows, label in ((1, "T=1"), (T0, f"T={T0}")):
        # T=512 at this width moves 2.7-18 MB per launch (0.3-2.3 us at peak): still the launch, not the stream
        note = "launch-bound"
        us = timed(lambda i: check(L.apk_embed_rows(h, apklib.FMT_Q8_0, p(q8), V0, H0, p(ids0[i % 8]), rows,
                                                    p(an0[i % len(an0)]["d"]), F32)), 200)
        record("embed_rows Q8_0->f32", f"qwen3-0.6b {label}", us, rows * (1088 + 4 + H0 * 4), note=note)
        us = timed(lambda i: check(L.apk_add_rmsnorm_rows(h, p(an0[i % len(an0)]["x"]), p(an0[i % len(an0)]["d"]),
                                                          p(an0[i % len(an0)]["h"]), p(g0), H0, rows, EPS, F32)), 200)
        record("add_rmsnorm", f"qwen3-0.6b {label} f32", us, 4 * rows * H0 * 4 + 4 * H0, note=note)
        us = timed(lambda i: check(L.apk_qknorm_rope_neox(h, p(qk0[i % len(qk0)]["q"]), p(qk0[i % len(qk0)]["k"]), p(qw), p(kw),
                                                          p(rope), rows, NQ0, NKV0, HD, HD, EPS, F32)), 200)
        record("qknorm_rope_neox", f"qwen3-0.6b {label} f32", us, 2 * rows * (NQ0 + NKV0) * HD * 4 + rows * (HD // 2) * 8 + 2 * HD * 4, note=note)
        us = timed(lambda i: check(L.apk_swiglu(h, p(sw0[i % len(sw0)]["gate"]), p(sw0[i % len(sw0)]["up"]), rows * FF0, F32)), 200)
        record("swiglu", f"qwen3-0.6b {label} f32", us, 3 * rows * FF0 * 4, note=note)
    del q8, an0, qk0, sw0

    # Qwen3-30B-A3B MoE layer ops, T=1024 tokens, f32 (config 4)
    mm = synth.MODELS["qwen3-30b-a3b"]
    TM, HM, NE, K, FM = 1024, mm["hidden"], mm["n_expert"], mm["top_k"], mm["moe_ffn"]
    logits = [randn((TM, NE), f32) for _ in range(8)]
    ga = pool(TM * HM * 4 + TM * K * HM * 4, lambda: dict(hs=randn((TM, HM), f32), xe=torch.empty((TM * K, HM), dtype=f32, device=dev)))
    # SwiGLU pools: 80 sets of 50 MB (the op-by-op chain below gates each of them once: 3 + 3 x 24 layers), every gate a copy of one pristine tensor that the timing restores them from
    gate_m = randn((TM * K, FM), f32)
    se = [dict(gate=gate_m.clone(), up=randn((TM * K, FM), f32)) for _ in range(80)]
    i32 = torch.int32
    ids_m = torch.empty((TM, K), dtype=i32, device=dev)
    w_m = torch.empty((TM, K), dtype=f32, device=dev)
    tbl = torch.zeros((NE, 3), dtype=i32, device=dev)
    n_used = torch.zeros(1, dtype=i32, device=dev)
    tok = torch.empty(TM * K, dtype=i32, device=dev)
    tok_off = torch.empty(TM + 1, dtype=i32, device=dev)
    hit_row = torch.empty(TM * K, dtype=i32, device=dev)
    hit_w = torch.empty(TM * K, dtype=f32, device=dev)
    torch.cuda.synchronize()
    tagm = f"qwen3-30b-a3b T={TM} f32"
    us = timed(lambda i: check(L.apk_route_topk(h, p(logits[i % 8]), None, TM, NE, K, 1, 1.0, 0, p(ids_m), p(w_m))), 200)
    record("route_topk", tagm, us, TM * NE * 4 + TM * K * 8, note="launch-bound")
    us = timed(lambda i: check(L.apk_moe_permute(h, p(ids_m), p(w_m), TM, K, NE, p(tbl), p(n_used), p(tok), p(tok_off),
                                                 p(hit_row), p(hit_w))), 200)
    record("moe_permute (tables)", tagm, us, TM * K * 8 + TM * K * 12 + TM * 4, note="launch-bound")
    # a decode step of the same router: one token, router and grouping as two launches and as one
    def two_launches(i):
        check(L.apk_route_topk(h, p(logits[i % 8]), None, 1, NE, K, 1, 1.0, 0, p(ids_m), p(w_m)))
        check(L.apk_moe_permute(h, p(ids_m), p(w_m), 1, K, NE, p(tbl), p(n_used), p(tok), p(tok_off), p(hit_row), p(hit_w)))
    us = timed(two_launches, 200)
    record("route_topk + moe_permute (two launches)", "qwen3-30b-a3b decode T=1 f32", us, NE * 4 + K * 28 + 8, launches=2, note="launch-bound")
    us = timed(lambda i: check(L.apk_route_group(h, p(logits[i % 8]), None, 1, NE, K, 1, 1.0, 0, p(ids_m), p(w_m), p(tbl), p(n_used),
                                                 p(tok), p(tok_off), p(hit_row), p(hit_w))), 200)
    record("route_group (router + grouping, one launch)", "qwen3-30b-a3b decode T=1 f32", us, NE * 4 + K * 28 + 8, note="launch-bound")
    us = timed(lambda i: check(L.apk_gather_rows(h, p(ga[i % len(ga)]["hs"]), p(tok), TM, TM * K, HM, p(ga[i % len(ga)]["xe"]), F32)), reps)
    record("gather_rows (permute, row-side)", tagm, us, TM * HM * 4 + TM * K * HM * 4 + TM * K * 4)
    us = timed(lambda i: check(L.apk_scatter_rows(h, p(ga[i % len(ga)]["hs"]), p(hit_row), TM, K, TM * K, HM, p(ga[i % len(ga)]["xe"]), F32)), reps)
    record("scatter_rows (permute, token-side)", tagm, us, TM * HM * 4 + TM * K * HM * 4 + TM * K * 4)
    us = timed(lambda i: check(L.apk_swiglu(h, p(se[i % len(se)]["gate"]), p(se[i % len(se)]["up"]), TM * K * FM, F32)), reps,
               refresh=lambda: restore_gates(se, gate_m), span=len(se))
    assert dead_fraction(se) < 0.01
    record("swiglu", f"qwen3-30b-a3b [{TM * K}x{FM}] f32", us, 3 * TM * K * FM * 4)
    # MoE combine + residual + next norm: the expert down rows [8192 x 2048] folded back into [1024 x 2048]
    cb = pool(TM * K * HM * 4 + 3 * TM * HM * 4, lambda: dict(flat=randn((TM * K, HM), f32), x=randn((TM, HM), f32),
                                                          h=torch.empty((TM, HM), dtype=f32, device=dev)))
    gm = 1 + 0.05 * randn(HM, f32)
    torch.cuda.synchronize()
    us = timed(lambda i: check(L.apk_moe_combine_add_rmsnorm(h, p(cb[i % len(cb)]["x"]), p(cb[i % len(cb)]["flat"]), p(tok_off), p(hit_row),
                                                             p(hit_w), TM * K, p(cb[i % len(cb)]["h"]), p(gm), HM, TM, EPS, F32)), reps)
    record("moe_combine + add + rmsnorm (one launch)", tagm, us, TM * K * HM * 4 + 3 * TM * HM * 4 + HM * 4 + TM * K * 8)
    # the five launches of one MoE layer in a row (router, grouping, token-side permute, SwiGLU on the grouped rows,
    # combine + residual + next norm), op by op and recorded once and replayed
    se2 = se  # one set per layer of a timed batch / of a replay, restored in between
    torch.cuda.synchronize()
    moe_bytes = (TM * NE * 4 + TM * K * 8) + (TM * K * 8 + TM * K * 12 + TM * 4) + (TM * HM * 4 + TM * K * HM * 4 + TM * K * 4) \
        + 3 * TM * K * FM * 4 + (TM * K * HM * 4 + 3 * TM * HM * 4 + HM * 4 + TM * K * 8)

    def moe_layer(i):
        check(L.apk_route_topk(h, p(logits[i % 8]), None, TM, NE, K, 1, 1.0, 0, p(ids_m), p(w_m)))
        check(L.apk_moe_permute(h, p(ids_m), p(w_m), TM, K, NE, p(tbl), p(n_used), p(tok), p(tok_off), p(hit_row), p(hit_w)))
        check(L.apk_scatter_rows(h, p(ga[i % len(ga)]["hs"]), p(hit_row), TM, K, TM * K, HM, p(ga[i % len(ga)]["xe"]), F32))
        check(L.apk_swiglu(h, p(se2[i % len(se2)]["gate"]), p(se2[i % len(se2)]["up"]), TM * K * FM, F32))
        check(L.apk_moe_combine_add_rmsnorm(h, p(cb[i % len(cb)]["x"]), p(cb[i % len(cb)]["flat"]), p(tok_off), p(hit_row), p(hit_w),
                                            TM * K, p(cb[i % len(cb)]["h"]), p(gm), HM, TM, EPS, F32))

    # Live gates without a restore inside the timed sequence: the pool is long enough for every layer of the op-by-op
    # timing (3 untimed + 3 x 24) to gate a set of its own, so the gates are restored once, ahead of it.  (Restoring
    # them ahead of every batch was tried and is not used: a batch that follows the restore of all sets ran 2.7 us per
    # layer slower, all of it in the scatter kernel and whether the restored data were activations or zeros.)
    check(L.apk_sync(h))
    restore_gates(se2, gate_m)
    torch.cuda.synchronize()
    record("MoE layer chain (router, grouping, permute, swiglu, combine+norm), op by op", tagm, timed(moe_layer, 24), moe_bytes, launches=5)
    assert dead_fraction(se2) < 0.01
    # recorded once (24 layers, a set of gates each) and replayed: restored gates, one untimed replay, three timed ones
    # (f32 gates stay activations over four applications: none reaches zero or the subnormal range)
    NREC = 24
    gmoe = C.c_void_p()
    check(L.apk_capture_begin(h))
    for i in range(3, 3 + NREC):
        moe_layer(i)
    check(L.apk_capture_end(h, C.byref(gmoe)))
    ms1, reps_us = C.c_float(), []
    for _ in range(5):
        check(L.apk_sync(h))
        restore_gates(se2, gate_m)
        torch.cuda.synchronize()
        check(L.apk_graph_launch(h, gmoe))
        check(L.apk_timer_begin(h))
        for _r in range(3):
            check(L.apk_graph_launch(h, gmoe))
        check(L.apk_timer_end(h, C.byref(ms1)))
        reps_us.append(ms1.value * 1000.0 / (3 * NREC))
    assert dead_fraction(se2) < 0.01
    record("MoE layer chain, recorded once and replayed", tagm, sorted(reps_us)[2], moe_bytes, launches=5)
    check(L.apk_graph_destroy(h, gmoe))
    del cb, se2, se
    # the same three streaming ops on fp16 activations (the reference's MoE path is f32; a second run at half the bytes,
    # same tables): every set of gates is gated once between two restores
    f16 = torch.float16
    tagh = f"qwen3-30b-a3b T={TM} f16"
    gh = pool(TM * HM * 2 + TM * K * HM * 2, lambda: dict(hs=randn((TM, HM)), xe=torch.empty((TM * K, HM), dtype=f16, device=dev)))
    us = timed(lambda i: check(L.apk_scatter_rows(h, p(gh[i % len(gh)]["hs"]), p(hit_row), TM, K, TM * K, HM, p(gh[i % len(gh)]["xe"]), F16)), reps)
    record("scatter_rows (permute, token-side)", tagh, us, TM * HM * 2 + TM * K * HM * 2 + TM * K * 4)
    del gh
    gate_h = randn((TM * K, FM))
    sh = [dict(gate=gate_h.clone(), up=randn((TM * K, FM))) for _ in range(max(6, int(COLD_BYTES // (2 * TM * K * FM * 2)) + 1))]
    us = timed(lambda i: check(L.apk_swiglu(h, p(sh[i % len(sh)]["gate"]), p(sh[i % len(sh)]["up"]), TM * K * FM, F16)), reps,
               refresh=lambda: restore_gates(sh, gate_h), span=len(sh))
    assert dead_fraction(sh) < 0.01
    record("swiglu", f"qwen3-30b-a3b [{TM * K}x{FM}] f16", us, 3 * TM * K * FM * 2)
    del sh
    ch = pool(TM * K * HM * 2 + 3 * TM * HM * 2, lambda: dict(flat=randn((TM * K, HM)), x=randn((TM, HM)),
                                                          h=torch.empty((TM, HM), dtype=f16, device=dev)))
    x_h = [s_["x"].clone() for s_ in ch]  # x += ... in place: restored between batches so that fp16 sums stay finite

    def restore_x():
        for s_, x0 in zip(ch, x_h):
            s_["x"].copy_(x0)

    torch.cuda.synchronize()
    us = timed(lambda i: check(L.apk_moe_combine_add_rmsnorm(h, p(ch[i % len(ch)]["x"]), p(ch[i % len(ch)]["flat"]), p(tok_off), p(hit_row),
                                                             p(hit_w), TM * K, p(ch[i % len(ch)]["h"]), p(gm), HM, TM, EPS, F16)), reps,
               refresh=restore_x)
    record("moe_combine + add + rmsnorm (one launch)", tagh, us, TM * K * HM * 2 + 3 * TM * HM * 2 + HM * 4 + TM * K * 8)
    del ch, x_h
    # greedy pick over the vocabulary (after the output head): 1 and 64 rows of 151936 logits
    V = synth.MODELS["qwen3-32b"]["vocab"]
    lg = [randn((64, V), f32) for _ in range(17)]  # 17 x 38.9 MB
    pick = torch.empty(64, dtype=i32, device=dev)
    torch.cuda.synchronize()
    for rows in (1, 64):
        us = timed(lambda i: check(L.apk_argmax_rows(h, p(lg[i % 17]), rows, V, p(pick))), 200)
        record("argmax_rows", f"{rows} x {V} logits f32", us, rows * V * 4 + rows * 4, note="launch-bound" if rows == 1 else None)
    del lg, ga
    # the plain-copy ceilings at the byte counts of the MoE layer's launches and of the greedy pick (a copy moves half
    # of the bytes in and half out; the pick only reads, which this library has no plain kernel for)
    cp_pool = torch.empty(int(COLD_BYTES * 1.1) // 4 * 4, dtype=torch.uint8, device=dev)
    cp_pool.view(torch.float32).normal_()  # not zeros: a stream of zeros runs 3-4 % faster than one of activations
    torch.cuda.synchronize()
    for name, nb in (("swiglu [8192x768] f32 and of scatter_rows", 3 * TM * K * FM * 4),
                     ("moe_combine + add + rmsnorm", TM * K * HM * 4 + 3 * TM * HM * 4 + HM * 4 + TM * K * 8),
                     ("argmax_rows 64 x 151936", 64 * V * 4)):
        half = nb // 2 // 4096 * 4096
        nset = cp_pool.numel() // (2 * half)
        us = timed(lambda i: check(L.apk_copy(h, p(cp_pool) + (i % nset) * 2 * half, p(cp_pool) + (i % nset) * 2 * half + half, half)), reps)
        record(f"copy (plain stream) of the bytes of {name}", f"{2 * half / 1e6:.1f} MB moved", us, 2 * half, note="ceiling at this size")
    # SwiGLU reads two streams and writes one; the same access mix with no arithmetic at all (a += b) is its nearer ceiling
    n_sw = TM * K * FM
    nset = cp_pool.numel() // (2 * n_sw * 4)
    us = timed(lambda i: check(L.apk_add_assign(h, p(cp_pool) + (i % nset) * 2 * n_sw * 4, p(cp_pool) + (i % nset) * 2 * n_sw * 4 + n_sw * 4, n_sw, F32)), reps)
    record("add_assign (two reads + one write, no arithmetic) at the size of swiglu [8192x768] f32", f"{3 * n_sw * 4 / 1e6:.1f} MB moved", us, 3 * n_sw * 4,
           note="ceiling of this access mix")
    del cp_pool


def cpu_baseline(np, lay, T, H, NQ, NKV, HD, FF, EPS):
    """The CPU oracle on the same layer chain and the same seeded inputs as the device leg (f32 activations: the
    reference's CPU path has no other), whole T rows, a few repetitions (~10-20 s)."""
    import oracle as ora

    ora.build()
    cores = os.cpu_count() or 1
    x, d, gamma = lay["x"].copy(), lay["delta"], lay["gamma1"]
    hbuf = np.empty_like(x)
    q, k, qw, kw = lay["q"].copy(), lay["k"].copy(), lay["qw"], lay["kw"]
    inv = ora.rope_inv_freq(HD, 1e6)
    ropes = ora.rope_table(list(range(T)), inv)
    gate, up = lay["gate"].copy(), lay["up"]

    def layer():
        ora.add_assign_par(x.reshape(-1), d.reshape(-1), cores)          # prefill.rs:246
        ora.rmsnorm_rows_into(hbuf.reshape(-1), x.reshape(-1), gamma, EPS, threads=cores)  # prefill.rs:155
        ora.qknorm_rope_rows(q, k, NQ, NKV, HD, qw, kw, ropes, EPS)      # attention.rs:131-165, serial
        ora.add_assign_par(x.reshape(-1), d.reshape(-1), cores)
        ora.rmsnorm_rows_into(hbuf.reshape(-1), x.reshape(-1), gamma, EPS, threads=cores)
        ora.swiglu(gate.reshape(-1), up.reshape(-1))                     # moe.rs:126, serial

    layer()  # warm-up
    times = []
    t_end = time.perf_counter() + 12.0
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 40):
        gate[:] = up  # keep SwiGLU inputs in a sane range across repetitions
        t0 = time.perf_counter()
        layer()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]

    def med_us(fn, reps=5):
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return round(sorted(ts)[len(ts) // 2] * 1e6, 1)

    # the same ops one by one, and the other ops of the path at their benchmark shapes (a few repetitions each)
    from allpaka_amd import synth
    per_op = {
        "add_assign + rmsnorm_rows_into (pool-parallel)": med_us(lambda: (ora.add_assign_par(x.reshape(-1), d.reshape(-1), cores),
                                                                          ora.rmsnorm_rows_into(hbuf.reshape(-1), x.reshape(-1), gamma, EPS, threads=cores))),
        "qknorm_rope rows (serial)": med_us(lambda: ora.qknorm_rope_rows(q, k, NQ, NKV, HD, qw, kw, ropes, EPS), 3),
        "swiglu (serial)": med_us(lambda: (gate.__setitem__(slice(None), up), ora.swiglu(gate.reshape(-1), up.reshape(-1))), 3),
    }
    gq = synth.rng(2, 1)
    table = synth.q4_k_table(gq, 4096, H)  # a slice of the vocabulary is enough for the CPU gather: rows are independent
    ids = gq.integers(0, 4096, size=T, dtype=np.uint32)
    per_op["embed_rows Q4_K (serial row_into loop)"] = med_us(lambda: ora.embed_rows(table, ora.FMT["Q4K"], 4096, H, ids), 3)
    logits = gq.standard_normal((1024, 128), dtype=np.float32)
    per_op["route_gated, 1024 tokens x 128 experts, k=8 (parallel over tokens)"] = med_us(lambda: ora.route_rows(logits, 8, ora.SOFTMAX, True, 1.0, threads=cores))
    rid, rw = ora.route_rows(logits, 8, ora.SOFTMAX, True, 1.0, threads=cores)
    per_op["grouping + CSR, 1024 tokens (serial)"] = med_us(lambda: ora.moe_group(rid, rw, 128))
    return {"value": round(med * 1e6, 1), "unit": "us/layer", "cores": cores, "kind": "port", "per_op_us": per_op,
            "sample": f"median of {len(times)} repetitions of the whole T={T} layer chain in f32 (the reference's CPU activations are f32); "
                      "C restatement of the reference CPU path, not the reference binary; residual add and row norms "
                      "pool-parallel, QK-norm+RoPE and SwiGLU serial, as the reference runs them"}


if __name__ == "__main__":
    main()

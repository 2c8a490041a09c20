"""The reference's whole-token request (gpu/types.rs:112-254: TokenReq, TokenLayer, TokenFfn) served with this
library's entries in the reference's call order, next to the same token on the CPU path.

What is under test is the mapping from request fields to entry arguments: raw F32 GGUF bytes as norm weights and
biases, `(sin, cos)` rows of `rot_dim / 2` pairs, K and V planes at ELEMENT offsets `k_off` / `v_off` of one shared
f16 cache region, rows stored at `pos .. pos + m`, the embedding row taken from `(embd, token_id)`, the router's
table / CSR feeding the combine, the NEXT layer's norm folded into the combine, the greedy pick.  The matmuls and
the attention over the cache, which this library does not have, are plain float32 products on both sides (torch on the
device, numpy on the host): they stand where a host's GEMM / attention provider would.  Tolerances are therefore
those of two float32 matmul implementations, not of the fused ops (which the other test files hold to their own bars).
"""
from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F32 = 8  # dq_fmt code of GgmlType::F32 (gpu/common.rs:47-61)
Q8_0 = 3


# ---- the request, field for field as in gpu/types.rs (the gated-delta-net and Gemma-only fields are left out) ----
@dataclass
class Dense:  # TokenFfn::Dense
    gate: tuple  # (ty, bytes, n_out)
    up: tuple
    down: tuple


@dataclass
class Moe:  # TokenFfn::Moe
    router: tuple  # (F32, bytes, n_expert)
    router_bias: Optional[bytes]
    gate: tuple  # (ty, bytes): packed [n_expert][expert_ffn][hidden]
    up: tuple
    down: tuple  # packed [n_expert][hidden][expert_ffn]
    expert_ffn: int
    n_used: int
    sigmoid: bool
    shared: Optional[list] = None  # [gate, up, down] as (ty, bytes, n_out)


@dataclass
class TokenLayer:
    attn_norm: bytes  # raw F32 bytes
    ffn_norm: bytes
    wq: tuple
    wk: tuple
    wv: tuple
    wo: tuple
    q_bias: Optional[bytes]
    k_bias: Optional[bytes]
    v_bias: Optional[bytes]
    q_norm: Optional[np.ndarray]
    k_norm: Optional[np.ndarray]
    k_off: int  # ELEMENT offsets into the cache region
    v_off: int
    ffn: object


@dataclass
class TokenReq:
    layers: list
    output_norm: bytes
    output: tuple
    embd: Optional[tuple]  # (ty, bytes, hidden)
    token_id: Optional[int]
    x: np.ndarray
    m: int
    rope: np.ndarray  # [m * rot_dim / 2][2] = (sin, cos)
    rot_dim: int
    rope_norm: bool
    eps: float
    cache: object  # the shared f16 region: a numpy u16 array on the host path, a device tensor on the GPU path
    cache_capacity: int
    kv_dim: int
    head_dim: int
    n_heads: int
    n_kv_heads: int
    pos: int
    scale: float
    argmax: bool
    norm_topk: bool = True
    hidden: int = field(default=0)


def f32s(raw, n):
    """norm_f32_bytes (gpu/cuda/attn.rs:254): raw little-endian F32 bytes of exactly n floats."""
    a = np.frombuffer(raw, dtype="<f4")
    assert a.size == n
    return np.ascontiguousarray(a)


def mat(w, n_in):
    ty, raw, n_out = w
    assert ty == F32
    return f32s(raw, n_out * n_in).reshape(n_out, n_in)


# ---- the CPU path: the reference's ops (through the checker) around numpy products ---------------------------------
def decode_token_cpu(ora, req):
    H, hd, nq, nkv, m = req.hidden, req.head_dim, req.n_heads, req.n_kv_heads, req.m
    kv, group = req.kv_dim, req.n_heads // req.n_kv_heads
    if req.embd is not None and req.token_id is not None and m == 1:
        ty, raw, hidden = req.embd
        vocab = len(raw) // ora.expected_bytes(ty, hidden)
        x = ora.embed_rows(np.frombuffer(raw, np.uint8), ty, vocab, hidden, np.array([req.token_id], np.uint32)).reshape(1, H)
    else:
        x = req.x.reshape(m, H).copy()
    rope_flat = np.ascontiguousarray(req.rope, np.float32).reshape(m, req.rot_dim // 2, 2)
    h = np.zeros_like(x)
    delta, normed = None, False
    caches = []
    for li, L in enumerate(req.layers):
        if not normed:
            ora.add_rmsnorm_rows(x, delta, h, f32s(L.attn_norm, H), req.eps)
        q = h @ mat(L.wq, H).T
        k = h @ mat(L.wk, H).T
        v = h @ mat(L.wv, H).T
        q, k, v = (np.ascontiguousarray(t, np.float32) for t in (q, k, v))
        if L.v_bias is not None:
            ora.add_bias_rows(v, f32s(L.v_bias, kv))
        ora.qknorm_rope_rows(q, k, nq, nkv, hd, L.q_norm, L.k_norm, rope_flat, req.eps, style=int(req.rope_norm),
                             q_bias=None if L.q_bias is None else f32s(L.q_bias, nq * hd),
                             k_bias=None if L.k_bias is None else f32s(L.k_bias, kv))
        kc = req.cache[L.k_off : L.k_off + req.cache_capacity * kv].reshape(req.cache_capacity, kv)
        vc = req.cache[L.v_off : L.v_off + req.cache_capacity * kv].reshape(req.cache_capacity, kv)
        ora.kv_store_rows(k, v, np.arange(req.pos, req.pos + m, dtype=np.uint32), kc, vc)
        caches.append((kc, vc))
        att = np.zeros((m, nq * hd), np.float32)
        for r in range(m):
            n_pos = req.pos + r + 1
            kf = ora.f16_bits_to_f32(kc[:n_pos].copy()).reshape(n_pos, nkv, hd)
            vf = ora.f16_bits_to_f32(vc[:n_pos].copy()).reshape(n_pos, nkv, hd)
            for hq in range(nq):
                s = (kf[:, hq // group, :] @ q[r, hq * hd : (hq + 1) * hd]) * np.float32(req.scale)
                p = np.exp(s - s.max())
                p /= p.sum()
                att[r, hq * hd : (hq + 1) * hd] = p @ vf[:, hq // group, :]
        o = np.ascontiguousarray(att @ mat(L.wo, nq * hd).T, np.float32)
        ora.add_rmsnorm_rows(x, o, h, f32s(L.ffn_norm, H), req.eps)
        nxt = f32s(req.layers[li + 1].attn_norm if li + 1 < len(req.layers) else req.output_norm, H)
        if isinstance(L.ffn, Dense):
            g = np.ascontiguousarray(h @ mat(L.ffn.gate, H).T, np.float32)
            u = np.ascontiguousarray(h @ mat(L.ffn.up, H).T, np.float32)
            ora.swiglu(g, u)
            delta = np.ascontiguousarray(g @ mat(L.ffn.down, g.shape[1]).T, np.float32)
            normed = False
        else:
            F = L.ffn
            E, ff = F.router[2], F.expert_ffn
            logits = np.ascontiguousarray(h @ mat(F.router, H).T, np.float32)
            bias = None if F.router_bias is None else f32s(F.router_bias, E)
            ids, w = ora.route_rows(logits, F.n_used, gating=ora.SIGMOID if F.sigmoid else ora.SOFTMAX, norm=req.norm_topk, scale=1.0, bias=bias)
            table, tok, tok_off, hit_row, hit_w = ora.moe_group(ids, w, E)
            total = int(tok.size)
            xe = ora.gather_rows(h, tok)
            Wg = f32s(F.gate[1], E * ff * H).reshape(E, ff, H)
            Wu = f32s(F.up[1], E * ff * H).reshape(E, ff, H)
            Wd = f32s(F.down[1], E * H * ff).reshape(E, H, ff)
            flat = np.zeros((total + (m if F.shared else 0), H), np.float32)
            for e, row0, rows in table:
                g = np.ascontiguousarray(xe[row0 : row0 + rows] @ Wg[e].T, np.float32)
                u = np.ascontiguousarray(xe[row0 : row0 + rows] @ Wu[e].T, np.float32)
                ora.swiglu(g, u)
                flat[row0 : row0 + rows] = g @ Wd[e].T
            if F.shared:
                sg, su, sd = F.shared
                g = np.ascontiguousarray(h @ mat(sg, H).T, np.float32)
                u = np.ascontiguousarray(h @ mat(su, H).T, np.float32)
                ora.swiglu(g, u)
                flat[total:] = g @ mat(sd, g.shape[1]).T
                tok_off, hit_row, hit_w = ora.moe_shared_hits(tok_off, hit_row, hit_w, total)
            ora.moe_combine_add_rmsnorm(x, flat, tok_off, hit_row, hit_w, h, nxt, req.eps)
            delta, normed = None, True
    if not normed:
        ora.add_rmsnorm_rows(x, delta, h, f32s(req.output_norm, H), req.eps)
    logits = np.ascontiguousarray(h @ mat(req.output, H).T, np.float32)
    return logits, h.copy(), [ora.argmax_last(logits[r]) for r in range(m)]


# ---- the same request through the library: every step that is not a product is one entry of the C ABI ----------------
def decode_token_gpu(be, req):
    import torch

    from allpaka_amd.backend import Gating, QuantMat

    dev = be.device
    H, hd, nq, nkv, m = req.hidden, req.head_dim, req.n_heads, req.n_kv_heads, req.m
    kv, group = req.kv_dim, req.n_heads // req.n_kv_heads
    up = lambda a: torch.from_numpy(np.array(a, copy=True, order="C")).to(dev)
    W = lambda w, n_in: up(mat(w, n_in))  # what resolve_w hands a GEMM provider
    if req.embd is not None and req.token_id is not None and m == 1:
        ty, raw, hidden = req.embd
        table = up(np.frombuffer(raw, np.uint8))
        x = torch.empty((1, H), dtype=torch.float32, device=dev)
        QuantMat(be, table, ty, len(raw) // be.L.apk_row_bytes(ty, hidden), hidden).row_into(req.token_id, x)  # apk_embed_rows_host_ids
    else:
        x = up(req.x.reshape(m, H))
    rope_flat = up(np.ascontiguousarray(req.rope, np.float32).reshape(m, req.rot_dim // 2, 2))  # the request's own layout
    cache_pos = up(np.arange(req.pos, req.pos + m, dtype=np.int32))
    h = torch.empty_like(x)
    delta, normed = None, False
    cache16 = req.cache.view(torch.float16)
    for li, L in enumerate(req.layers):
        if not normed:
            be.add_rmsnorm_rows(x, delta, h, up(f32s(L.attn_norm, H)), req.eps)
        q = (h @ W(L.wq, H).T).contiguous()
        k = (h @ W(L.wk, H).T).contiguous()
        v = (h @ W(L.wv, H).T).contiguous()
        # K and V planes of this layer: element offsets into the one f16 region
        kc = cache16[L.k_off : L.k_off + req.cache_capacity * kv].view(req.cache_capacity, kv)
        vc = cache16[L.v_off : L.v_off + req.cache_capacity * kv].view(req.cache_capacity, kv)
        be.attn_prologue_rows(q, k, v, nq, nkv, hd, req.eps, rope_flat,
                              q_bias=None if L.q_bias is None else up(f32s(L.q_bias, nq * hd)),
                              k_bias=None if L.k_bias is None else up(f32s(L.k_bias, kv)),
                              v_bias=None if L.v_bias is None else up(f32s(L.v_bias, kv)),
                              q_norm=None if L.q_norm is None else up(L.q_norm), k_norm=None if L.k_norm is None else up(L.k_norm),
                              cache_pos=cache_pos, k_cache=kc, v_cache=vc, adjacent_pairs=req.rope_norm, rot_dim=req.rot_dim)
        att = torch.zeros((m, nq * hd), dtype=torch.float32, device=dev)
        for r in range(m):  # [ATTN]
            n_pos = req.pos + r + 1
            kf = kc[:n_pos].float().view(n_pos, nkv, hd).repeat_interleave(group, dim=1)
            vf = vc[:n_pos].float().view(n_pos, nkv, hd).repeat_interleave(group, dim=1)
            s = torch.einsum("phd,hd->hp", kf, q[r].view(nq, hd)) * req.scale
            att[r] = torch.einsum("hp,phd->hd", torch.softmax(s, dim=1), vf).reshape(-1)
        o = (att @ W(L.wo, nq * hd).T).contiguous()
        be.add_rmsnorm_rows(x, o, h, up(f32s(L.ffn_norm, H)), req.eps)
        nxt = up(f32s(req.layers[li + 1].attn_norm if li + 1 < len(req.layers) else req.output_norm, H))
        if isinstance(L.ffn, Dense):
            g = (h @ W(L.ffn.gate, H).T).contiguous()
            u = (h @ W(L.ffn.up, H).T).contiguous()
            be.swiglu(g, u)
            delta = (g @ W(L.ffn.down, g.shape[1]).T).contiguous()
            normed = False
        else:
            F = L.ffn
            E, ff = F.router[2], F.expert_ffn
            logits = (h @ W(F.router, H).T).contiguous()
            bias = None if F.router_bias is None else up(f32s(F.router_bias, E))
            _, (table, tok, tok_off, hit_row, hit_w) = be.route_group(logits, F.n_used, gating=Gating.Sigmoid if F.sigmoid else Gating.Softmax,
                                                                      norm=req.norm_topk, scale=1.0, bias=bias)
            total = tok.numel()
            xe = be.scatter_rows(h, hit_row, F.n_used)  # the token-side permute: xe[hit_row[t*k + j]] = h[t]
            Wg = up(f32s(F.gate[1], E * ff * H).reshape(E, ff, H))
            Wu = up(f32s(F.up[1], E * ff * H).reshape(E, ff, H))
            Wd = up(f32s(F.down[1], E * H * ff).reshape(E, H, ff))
            flat = torch.zeros((total + (m if F.shared else 0), H), dtype=torch.float32, device=dev)
            for e, row0, rows in table.tolist():  # [GEMM] per group, the SwiGLU between them over the group's rows
                g = (xe[row0 : row0 + rows] @ Wg[e].T).contiguous()
                u = (xe[row0 : row0 + rows] @ Wu[e].T).contiguous()
                be.swiglu(g, u)
                flat[row0 : row0 + rows] = g @ Wd[e].T
            if F.shared:
                sg, su, sd = F.shared
                g = (h @ W(sg, H).T).contiguous()
                u = (h @ W(su, H).T).contiguous()
                be.swiglu(g, u)
                flat[total:] = g @ W(sd, g.shape[1]).T
                tok_off, hit_row, hit_w = be.moe_shared_hits(tok_off, hit_row, hit_w, total)
            be.moe_combine_add_rmsnorm(x, flat, tok_off, hit_row, hit_w, h, nxt, req.eps)  # the next layer's norm rides along
            delta, normed = None, True
    if not normed:
        be.add_rmsnorm_rows(x, delta, h, up(f32s(req.output_norm, H)), req.eps)
    logits = (h @ W(req.output, H).T).contiguous()
    picks = be.argmax_rows(logits) if req.argmax else None
    return logits.cpu().numpy(), h.cpu().numpy(), None if picks is None else picks.tolist()


def build_request(g, *, m, pos, token_id, rope_norm, rot_dim, biases, qk_norm, moe_shared, sigmoid):
    from allpaka_amd import synth

    H, hd, nq, nkv, ffn, vocab, E, k_used, eff, cap = 256, 64, 4, 2, 512, 96, 8, 2, 128, 32
    kv = nkv * hd
    raw = lambda a: np.ascontiguousarray(a, "<f4").tobytes()
    wmat = lambda n_out, n_in: (F32, raw(synth.normal_f32(g, (n_out, n_in), 0.0, 1.0 / np.sqrt(n_in))), n_out)
    gamma = lambda n: raw(synth.normal_f32(g, n, 1.0, 0.1))
    n_layers = 3
    layers = []
    for li in range(n_layers):
        if li == 1:
            ffn_ = Moe(router=wmat(E, H), router_bias=raw(synth.normal_f32(g, E, 0.0, 0.05)) if sigmoid else None,
                       gate=(F32, raw(synth.normal_f32(g, (E, eff, H), 0.0, 1.0 / 16))), up=(F32, raw(synth.normal_f32(g, (E, eff, H), 0.0, 1.0 / 16))),
                       down=(F32, raw(synth.normal_f32(g, (E, H, eff), 0.0, 1.0 / 11))), expert_ffn=eff, n_used=k_used, sigmoid=sigmoid,
                       shared=[wmat(eff, H), wmat(eff, H), wmat(H, eff)] if moe_shared else None)
        else:
            ffn_ = Dense(gate=wmat(ffn, H), up=wmat(ffn, H), down=wmat(H, ffn))
        layers.append(TokenLayer(
            attn_norm=gamma(H), ffn_norm=gamma(H), wq=wmat(nq * hd, H), wk=wmat(kv, H), wv=wmat(kv, H), wo=wmat(H, nq * hd),
            q_bias=raw(synth.normal_f32(g, nq * hd, 0.0, 0.1)) if biases else None, k_bias=raw(synth.normal_f32(g, kv, 0.0, 0.1)) if biases else None,
            v_bias=raw(synth.normal_f32(g, kv, 0.0, 0.1)) if biases else None,
            q_norm=synth.normal_f32(g, hd, 1.0, 0.1) if qk_norm else None, k_norm=synth.normal_f32(g, hd, 1.0, 0.1) if qk_norm else None,
            k_off=li * 2 * cap * kv, v_off=li * 2 * cap * kv + cap * kv, ffn=ffn_))
    import oracle as ora

    inv = ora.rope_inv_freq(rot_dim, 10000.0)
    rope = ora.rope_table(np.arange(pos, pos + m, dtype=np.uint32), inv).reshape(m * rot_dim // 2, 2)
    embd = (Q8_0, synth.q8_0_table(g, vocab, H).tobytes(), H)
    # a cache that already holds `pos` earlier positions of every layer (f16 bits), the rest zero
    cache = np.zeros(n_layers * 2 * cap * kv, np.uint16)
    for L in layers:
        for off in (L.k_off, L.v_off):
            cache[off : off + pos * kv] = synth.to_f16_bits(synth.normal_f32(g, pos * kv, 0.0, 0.5))
    return TokenReq(layers=layers, output_norm=gamma(H), output=wmat(vocab, H), embd=embd if m == 1 else None, token_id=token_id if m == 1 else None,
                    x=synth.normal_f32(g, m * H, 0.0, 1.0), m=m, rope=rope, rot_dim=rot_dim, rope_norm=rope_norm, eps=1e-6, cache=cache,
                    cache_capacity=cap, kv_dim=kv, head_dim=hd, n_heads=nq, n_kv_heads=nkv, pos=pos, scale=1.0 / np.sqrt(hd), argmax=True, hidden=H)


@pytest.mark.parametrize("case", [
    dict(m=1, pos=0, token_id=0, rope_norm=False, rot_dim=64, biases=False, qk_norm=True, moe_shared=False, sigmoid=False),   # Qwen3 style, first token
    dict(m=1, pos=7, token_id=95, rope_norm=False, rot_dim=64, biases=False, qk_norm=True, moe_shared=False, sigmoid=False),  # into a filled cache
    dict(m=4, pos=5, token_id=None, rope_norm=False, rot_dim=64, biases=False, qk_norm=True, moe_shared=False, sigmoid=False),  # verify rows (m > 1)
    dict(m=1, pos=3, token_id=17, rope_norm=True, rot_dim=64, biases=True, qk_norm=False, moe_shared=False, sigmoid=False),   # Llama / Qwen2 style
    dict(m=3, pos=9, token_id=None, rope_norm=False, rot_dim=32, biases=True, qk_norm=False, moe_shared=True, sigmoid=True),  # GLM style: partial rotary, sigmoid + bias, shared expert
])
def test_token_request_through_the_library_matches_the_cpu_path(case):
    import torch

    import oracle as ora
    from allpaka_amd import synth
    from allpaka_amd.backend import Backend

    ora.build()
    g = synth.rng(4, 1000 + 17 * case["m"] + case["pos"])
    req = build_request(g, **case)
    host_cache = req.cache.copy()
    req.cache = host_cache
    want_logits, want_h, want_pick = decode_token_cpu(ora, req)

    be = Backend(0)
    try:
        dev_req = build_request(synth.rng(4, 1000 + 17 * case["m"] + case["pos"]), **case)  # the same request, drawn again
        dev_req.cache = torch.from_numpy(dev_req.cache.view(np.int16).copy()).to(be.device)  # gpu::wrap_region: the region on the device
        got_logits, got_h, got_pick = decode_token_gpu(be, dev_req)
        assert be.take_faults() == 0
        cache_after = dev_req.cache.cpu().numpy().view(np.uint16)
    finally:
        be.close()
    # the cache: the rows pos .. pos + m of every layer's planes were written (others untouched), to within one code of
    # fp16 where the two float32 projections in front differ in their last bits
    kv, cap = req.kv_dim, req.cache_capacity
    before = build_request(synth.rng(4, 1000 + 17 * case["m"] + case["pos"]), **case).cache
    for L in req.layers:
        for off in (L.k_off, L.v_off):
            lo, hi = off + req.pos * kv, off + (req.pos + req.m) * kv
            assert np.array_equal(cache_after[off:lo], before[off:lo]) and np.array_equal(cache_after[hi : off + cap * kv], before[hi : off + cap * kv])
            assert np.any(cache_after[lo:hi] != 0)
            # codes differ by at most a few where the value is tiny next to the row's scale; compare as numbers
            a = ora.f16_bits_to_f32(cache_after[lo:hi].copy())
            b = ora.f16_bits_to_f32(host_cache[lo:hi].copy())
            assert np.max(np.abs(a - b)) <= 2e-3 * max(1.0, float(np.max(np.abs(b))))
    # measured: 2e-6 .. 2e-4 of the logits' scale (the larger figures where one cached value lands on the other fp16 code)
    scale = float(np.sqrt(np.mean(want_logits.astype(np.float64) ** 2)))
    assert np.max(np.abs(got_logits - want_logits)) <= 2e-3 * scale, np.max(np.abs(got_logits - want_logits)) / scale
    assert np.max(np.abs(got_h - want_h)) <= 2e-3 * float(np.sqrt(np.mean(want_h.astype(np.float64) ** 2)))
    # the greedy pick: the same token wherever the CPU's own top two are further apart than the products' noise
    for r in range(req.m):
        top = np.sort(want_logits[r])[-2:]
        if top[1] - top[0] > 1e-2 * scale:
            assert got_pick[r] == want_pick[r]
        assert got_pick[r] == int(np.flatnonzero(got_logits[r] == got_logits[r].max())[-1])  # and always its own logits' last maximum


# ---- a batched decode step: PrefillAttnReq with `multi` and `fusion`, then GroupedFfnReq with host-built lists ---------
def test_batched_decode_step_with_one_cache_per_session():
    """gpu/types.rs:302-365 and :406-467.  Row i is one token of session i: its K/V go to `multi[i].cache` at
    `multi[i].pos` and it attends over that cache's first pos + 1 positions (MultiRow); `fusion` supplies the two norms
    and the router; the positions are staged on the device and the rotary rows are built there from them
    (multi_stage with set_rope_inv_freq done).  The routed FFN then gets `groups`, `tok` and the CSR lists from the HOST
    (the reference's CUDA arm rebuilds them on the host from the downloaded logits, gpu/cuda/ffn_grouped.rs:22-120), gathers
    row-side, and folds `fused.next_norm` into the combine."""
    import torch

    import oracle as ora
    from allpaka_amd import synth
    from allpaka_amd.backend import Backend

    ora.build()
    g = synth.rng(4, 4242)
    H, hd, nq, nkv, E, k_used, eff, cap, eps = 256, 64, 4, 2, 8, 2, 128, 16, 1e-6
    kv, group, m = nkv * hd, nq // nkv, 3
    positions = np.array([5, 0, 11], np.uint32)  # each session at its own position
    nf = lambda shape, std=1.0, mean=0.0: synth.normal_f32(g, shape, mean, std)
    wq, wk, wv, wo = nf((nq * hd, H), 1 / 16), nf((kv, H), 1 / 16), nf((kv, H), 1 / 16), nf((H, nq * hd), 1 / 16)
    attn_norm, ffn_norm, next_norm = nf(H, 0.1, 1.0), nf(H, 0.1, 1.0), nf(H, 0.1, 1.0)
    q_norm, k_norm = nf(hd, 0.1, 1.0), nf(hd, 0.1, 1.0)
    router = nf((E, H), 1 / 16)
    Wg, Wu, Wd = nf((E, eff, H), 1 / 16), nf((E, eff, H), 1 / 16), nf((E, H, eff), 1 / 11)
    x0 = nf((m, H))
    # one cache region per session: [K plane | V plane], each [cap][kv] f16, filled up to the session's position
    caches = []
    for p in positions:
        c = np.zeros(2 * cap * kv, np.uint16)
        for off in (0, cap * kv):
            c[off : off + int(p) * kv] = synth.to_f16_bits(nf(int(p) * kv, 0.5))
        caches.append(c)
    inv = ora.rope_inv_freq(hd, 1e6)
    scale = 1.0 / np.sqrt(hd)

    # ---------------- CPU path
    x = x0.copy()
    h = np.zeros_like(x)
    ora.add_rmsnorm_rows(x, None, h, attn_norm, eps)
    q, k, v = (np.ascontiguousarray(h @ w.T, np.float32) for w in (wq, wk, wv))
    ropes = ora.rope_table(positions, inv)  # PrefillAttnReq.ropes: m * rot_dim / 2 (sin, cos) pairs
    ora.qknorm_rope_rows(q, k, nq, nkv, hd, q_norm, k_norm, ropes, eps)
    host_caches = [c.copy() for c in caches]
    att = np.zeros((m, nq * hd), np.float32)
    for i in range(m):
        kc, vc = host_caches[i][: cap * kv].reshape(cap, kv), host_caches[i][cap * kv :].reshape(cap, kv)
        ora.kv_store_rows(k[i : i + 1], v[i : i + 1], positions[i : i + 1], kc, vc)
        n_pos = int(positions[i]) + 1
        kf = ora.f16_bits_to_f32(kc[:n_pos].copy()).reshape(n_pos, nkv, hd)
        vf = ora.f16_bits_to_f32(vc[:n_pos].copy()).reshape(n_pos, nkv, hd)
        for hq in range(nq):
            s = (kf[:, hq // group, :] @ q[i, hq * hd : (hq + 1) * hd]) * np.float32(scale)
            pr = np.exp(s - s.max())
            pr /= pr.sum()
            att[i, hq * hd : (hq + 1) * hd] = pr @ vf[:, hq // group, :]
    ora.add_rmsnorm_rows(x, np.ascontiguousarray(att @ wo.T, np.float32), h, ffn_norm, eps)
    logits = np.ascontiguousarray(h @ router.T, np.float32)
    ids, w = ora.route_rows(logits, k_used, norm=True)
    groups, tok, tok_off, hit_row, hit_w = ora.moe_group(ids, w, E)  # GroupedFfnReq.groups / tok, GroupedCombine lists
    xe = ora.gather_rows(h, tok)
    flat = np.zeros((tok.size, H), np.float32)
    for e, row0, rows in groups:
        gg = np.ascontiguousarray(xe[row0 : row0 + rows] @ Wg[e].T, np.float32)
        uu = np.ascontiguousarray(xe[row0 : row0 + rows] @ Wu[e].T, np.float32)
        ora.swiglu(gg, uu)
        flat[row0 : row0 + rows] = gg @ Wd[e].T
    ora.moe_combine_add_rmsnorm(x, flat, tok_off, hit_row, hit_w, h, next_norm, eps)
    want_x, want_h = x, h

    # ---------------- the same step through the library
    be = Backend(0)
    try:
        dev = be.device
        up = lambda a: torch.from_numpy(np.array(a, copy=True, order="C")).to(dev)
        x = up(x0)
        h = torch.empty_like(x)
        be.add_rmsnorm_rows(x, None, h, up(attn_norm), eps)  # fusion.attn_norm over the resident residual rows
        q, k, v = ((h @ up(w).T).contiguous() for w in (wq, wk, wv))
        pos_dev = up(positions.view(np.int32))  # multi_stage: the positions, staged once for the step
        table = be.rope_table(pos_dev, up(inv))  # ... and the rotary rows built from them on the device
        assert np.max(np.abs(table.cpu().numpy().reshape(ropes.shape) - ropes)) <= 1e-6
        regions = [up(c.view(np.int16)).view(torch.float16) for c in caches]  # gpu::wrap_region of every session's cache
        att = torch.zeros((m, nq * hd), dtype=torch.float32, device=dev)
        for i in range(m):  # one call per distinct (cache, k_off, v_off): here one row each
            kc, vc = regions[i][: cap * kv].view(cap, kv), regions[i][cap * kv :].view(cap, kv)
            be.attn_prologue_rows(q[i : i + 1], k[i : i + 1], v[i : i + 1], nq, nkv, hd, eps, table[i : i + 1], q_norm=up(q_norm), k_norm=up(k_norm),
                                  cache_pos=pos_dev[i : i + 1], k_cache=kc, v_cache=vc)
            n_pos = int(positions[i]) + 1
            kf = kc[:n_pos].float().view(n_pos, nkv, hd).repeat_interleave(group, dim=1)
            vf = vc[:n_pos].float().view(n_pos, nkv, hd).repeat_interleave(group, dim=1)
            s = torch.einsum("phd,hd->hp", kf, q[i].view(nq, hd)) * scale
            att[i] = torch.einsum("hp,phd->hd", torch.softmax(s, dim=1), vf).reshape(-1)
        be.add_rmsnorm_rows(x, (att @ up(wo).T).contiguous(), h, up(ffn_norm), eps)  # fusion.ffn_norm
        dev_logits = (h @ up(router).T).contiguous()  # fusion.router: what prefill_attn_block returns
        # the host builds the lists from the downloaded logits, as the reference's CUDA arm does, and hands them over
        ids_h, w_h = ora.route_rows(dev_logits.cpu().numpy(), k_used, norm=True)
        groups_h, tok_h, tok_off_h, hit_row_h, hit_w_h = ora.moe_group(ids_h, w_h, E)
        assert np.array_equal(ids_h, ids)  # the same experts as on the CPU path (the logits differ in their last bits only)
        tok_d = up(tok_h.view(np.int32))
        xe = be.gather_rows(h, tok_d)  # GroupedFfnReq.x / tok: the row-side permute
        flat = torch.zeros((tok_h.size, H), dtype=torch.float32, device=dev)
        for e, row0, rows in groups_h.tolist():
            gg = (xe[row0 : row0 + rows] @ up(Wg[e]).T).contiguous()
            uu = (xe[row0 : row0 + rows] @ up(Wu[e]).T).contiguous()
            be.swiglu(gg, uu)
            flat[row0 : row0 + rows] = gg @ up(Wd[e]).T
        be.moe_combine_add_rmsnorm(x, flat, up(tok_off_h.view(np.int32)), up(hit_row_h.view(np.int32)), up(hit_w_h), h, up(next_norm), eps)
        assert be.take_faults() == 0
        got_x, got_h = x.cpu().numpy(), h.cpu().numpy()
        got_caches = [r.view(torch.int16).cpu().numpy().view(np.uint16) for r in regions]
    finally:
        be.close()
    for i in range(m):  # each session's cache: one new row at its own position, nothing else touched
        for off in (0, cap * kv):
            lo, hi = off + int(positions[i]) * kv, off + (int(positions[i]) + 1) * kv
            assert np.array_equal(got_caches[i][off:lo], caches[i][off:lo]) and np.array_equal(got_caches[i][hi : off + cap * kv], caches[i][hi : off + cap * kv])
            a, b = ora.f16_bits_to_f32(got_caches[i][lo:hi].copy()), ora.f16_bits_to_f32(host_caches[i][lo:hi].copy())
            assert np.any(got_caches[i][lo:hi] != 0) and np.max(np.abs(a - b)) <= 2e-3 * max(1.0, float(np.max(np.abs(b))))
    rms = lambda a: float(np.sqrt(np.mean(a.astype(np.float64) ** 2)))
    assert np.max(np.abs(got_x - want_x)) <= 2e-3 * rms(want_x)
    assert np.max(np.abs(got_h - want_h)) <= 2e-3 * rms(want_h)

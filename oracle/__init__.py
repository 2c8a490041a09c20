"""ctypes front-end of the CPU oracle (oracle/apk_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg -- never by the allpaka_amd package.  Arrays are
numpy, modified in place exactly where the reference modifies its slices.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")

FMT = {"Q4K": 0, "Q5K": 1, "Q6K": 2, "Q8_0": 3, "Q2K": 4, "Q3K": 5, "Q5_0": 6, "F16": 7, "F32": 8, "BF16": 9}


def build(force=False):
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "apk_oracle.c")):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "liboracle.so"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        sz, u32, i32, f32 = C.c_size_t, C.c_uint32, C.c_int, C.c_float
        vp = C.c_void_p
        L.ora_f16_to_f32.restype = f32
        L.ora_f16_to_f32.argtypes = [C.c_uint16]
        L.ora_f32_to_f16.restype = C.c_uint16
        L.ora_f32_to_f16.argtypes = [f32]
        L.ora_bf16_to_f32.restype = f32
        L.ora_bf16_to_f32.argtypes = [C.c_uint16]
        L.ora_f16_to_f32_slice.argtypes = [vp, vp, sz]
        L.ora_f32_to_f16_slice.argtypes = [vp, vp, sz]
        L.ora_scale_min_k4.argtypes = [i32, vp, vp, vp]
        L.ora_expected_bytes.restype = C.c_int64
        L.ora_expected_bytes.argtypes = [i32, sz]
        L.ora_embed_row_groups.restype = u32
        L.ora_embed_row_groups.argtypes = [u32, sz]
        L.ora_dequant_into.argtypes = [i32, vp, sz, vp, sz]
        L.ora_quantmat_row_into.argtypes = [vp, sz, i32, sz, sz, sz, vp, sz]
        L.ora_embed_rows.argtypes = [vp, sz, i32, sz, sz, vp, sz, vp]
        L.ora_embed_rows_f16.argtypes = [vp, sz, i32, sz, sz, vp, sz, vp]
        L.ora_sum_sq_f64.restype = C.c_double
        L.ora_sum_sq_f64.argtypes = [vp, sz]
        L.ora_rmsnorm.argtypes = [vp, vp, sz, f32]
        L.ora_rmsnorm_into.argtypes = [vp, vp, vp, sz, f32]
        L.ora_rmsnorm_rows_into.argtypes = [vp, sz, vp, sz, vp, sz, f32, sz]
        L.ora_add_assign_slice.argtypes = [vp, sz, vp, sz]
        L.ora_add_bias_rows.argtypes = [vp, sz, vp, sz]
        L.ora_add_bias_rows.restype = None
        L.ora_moe_shared_hits.argtypes = [vp, vp, vp, sz, sz, vp, vp, vp]
        L.ora_moe_shared_hits.restype = None
        L.ora_add_assign_par.argtypes = [vp, sz, vp, sz, sz]
        L.ora_add_scaled_slice.argtypes = [vp, sz, vp, sz, f32]
        L.ora_rope_inv_freq.argtypes = [sz, f32, vp]
        L.ora_rope_sin_cos.argtypes = [u32, vp, sz, vp]
        L.ora_rope_neox_cached_from_array.argtypes = [vp, sz, vp, sz]
        L.ora_rope_norm_cached_from_array.argtypes = [vp, sz, vp, sz]
        L.ora_rope_neox.argtypes = [vp, sz, u32, f32]
        L.ora_rope_norm.argtypes = [vp, sz, u32, f32]
        L.ora_qknorm_rope_rows.argtypes = [vp, vp, sz, sz, sz, sz, vp, vp, vp, sz, f32]
        L.ora_qknorm_rope_rows_f16.argtypes = [vp, vp, sz, sz, sz, sz, vp, vp, vp, sz, f32]
        L.ora_qknorm_rope_rows_style.argtypes = [vp, vp, sz, sz, sz, sz, vp, vp, vp, sz, f32, C.c_int]
        L.ora_qknorm_rope_rows_style_f16.argtypes = [vp, vp, sz, sz, sz, sz, vp, vp, vp, sz, f32, C.c_int]
        L.ora_silu.restype = f32
        L.ora_silu.argtypes = [f32]
        L.ora_swiglu.argtypes = [vp, sz, vp, sz]
        L.ora_swiglu_f16.argtypes = [vp, vp, sz]
        L.ora_geglu_tanh.argtypes = [vp, sz, vp, sz]
        L.ora_geglu_tanh_f16.argtypes = [vp, vp, sz]
        L.ora_gelu_tanh_mul.restype = f32
        L.ora_gelu_tanh_mul.argtypes = [f32, f32]
        L.ora_softmax.argtypes = [vp, sz]
        L.ora_sigmoid.argtypes = [vp, sz]
        L.ora_route_gated.restype = sz
        L.ora_route_gated.argtypes = [vp, sz, sz, i32, i32, f32, vp, vp, vp]
        L.ora_topk_by_logits.restype = sz
        L.ora_topk_by_logits.argtypes = [vp, sz, sz, vp]
        L.ora_route.restype = sz
        L.ora_route.argtypes = [vp, sz, sz, vp, vp]
        L.ora_route_rows.argtypes = [vp, sz, sz, sz, i32, i32, f32, vp, vp, vp, sz]
        L.ora_moe_group.restype = sz
        L.ora_moe_group.argtypes = [vp, vp, sz, sz, sz, vp, vp, vp, vp, vp]
        L.ora_gather_rows.argtypes = [vp, vp, sz, sz, vp]
        L.ora_gather_rows_f16.argtypes = [vp, vp, sz, sz, vp]
        L.ora_moe_combine_add_rmsnorm.argtypes = [vp, vp, vp, vp, vp, vp, vp, sz, sz, f32]
        L.ora_moe_combine_add_rmsnorm_f16.argtypes = [vp, vp, vp, vp, vp, vp, vp, sz, sz, f32]
        L.ora_argmax_last.restype = u32
        L.ora_argmax_last.argtypes = [vp, sz]
        L.ora_kv_store_rows.argtypes = [vp, vp, sz, sz, vp, sz, vp, vp]
        L.ora_kv_store_rows_f16.argtypes = [vp, vp, sz, sz, vp, sz, vp, vp]
        L.ora_add_rmsnorm_rows.argtypes = [vp, vp, vp, vp, sz, sz, f32]
        L.ora_add_rmsnorm_rows_f16.argtypes = [vp, vp, vp, vp, sz, sz, f32]
        _lib = L
    return _lib


def _p(a):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "oracle wants C-contiguous numpy arrays"
    return a.ctypes.data


def _chk(a, dt):
    assert a.dtype == np.dtype(dt), f"expected {dt}, got {a.dtype}"
    return a


class OracleError(Exception):
    """Stands for the reference's panic / Err at the same spot."""


# ---- dtype
def f16_to_f32(h):
    return float(lib().ora_f16_to_f32(int(h) & 0xFFFF))


def f32_to_f16(x):
    return int(lib().ora_f32_to_f16(float(np.float32(x))))


def f16_bits_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().ora_f16_to_f32_slice(_p(h), _p(out), h.size)
    return out


def f32_to_f16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().ora_f32_to_f16_slice(_p(x), _p(out), x.size)
    return out


def scale_min_k4(j, packed):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    sc, mn = C.c_float(), C.c_float()
    lib().ora_scale_min_k4(j, _p(packed), C.addressof(sc), C.addressof(mn))
    return sc.value, mn.value


def expected_bytes(fmt, elements):
    r = lib().ora_expected_bytes(fmt, elements)
    return None if r < 0 else int(r)


def embed_row_groups(fmt, n_in):
    return int(lib().ora_embed_row_groups(fmt, n_in))


# ---- dequant / embedding
def dequant(fmt, data, elements):
    data = np.ascontiguousarray(data, dtype=np.uint8)
    out = np.zeros(elements, np.float32)
    if lib().ora_dequant_into(fmt, _p(data), data.size, _p(out), elements):
        raise OracleError("GgufError::Dequant")
    return out


def quantmat_row(data, fmt, n_out, n_in, j, dst_len=None):
    data = np.ascontiguousarray(data, dtype=np.uint8)
    dst = np.zeros(n_in if dst_len is None else dst_len, np.float32)
    rc = lib().ora_quantmat_row_into(_p(data), data.size, fmt, n_out, n_in, j, _p(dst), dst.size)
    if rc:
        raise OracleError({1: "dequant", 2: "QuantMat::new bails", 3: "row out of range", 4: "dst length"}[rc])
    return dst


def embed_rows(data, fmt, vocab, n_in, ids, out_f16=False, scale=1.0):
    """QuantMat::row_into over ids; scale != 1: the `*v *= embed_scale` of model/prefill.rs:107-109
    (one f32 multiply per element after the dequant), then the optional narrowing to fp16."""
    data = np.ascontiguousarray(data, dtype=np.uint8)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    if scale != 1.0:
        rows = embed_rows(data, fmt, vocab, n_in, ids) * np.float32(scale)
        return f32_to_f16_bits(rows) if out_f16 else rows
    out = np.zeros((ids.size, n_in), np.uint16 if out_f16 else np.float32)
    fn = lib().ora_embed_rows_f16 if out_f16 else lib().ora_embed_rows
    rc = fn(_p(data), data.size, fmt, vocab, n_in, _p(ids), ids.size, _p(out))
    if rc:
        raise OracleError(f"embed_rows rc={rc}")
    return out


# ---- norm / residual
def sum_sq_f64(x):
    _chk(x, np.float32)
    return float(lib().ora_sum_sq_f64(_p(x), x.size))


def rmsnorm(x, w, eps):
    _chk(x, np.float32), _chk(w, np.float32)
    if x.size != w.size:
        raise OracleError("assert_eq!(x.len(), weight.len())")
    lib().ora_rmsnorm(_p(x), _p(w), x.size, eps)


def rmsnorm_into(dst, src, w, eps):
    for a in (dst, src, w):
        _chk(a, np.float32)
    if src.size != w.size or dst.size != src.size:
        raise OracleError("length assert")
    lib().ora_rmsnorm_into(_p(dst), _p(src), _p(w), src.size, eps)


def rmsnorm_rows_into(dst, src, w, eps, threads=1):
    for a in (dst, src, w):
        _chk(a, np.float32)
    if lib().ora_rmsnorm_rows_into(_p(dst), dst.size, _p(src), src.size, _p(w), w.size, eps, threads):
        raise OracleError("dst holds fewer rows than src")


def add_assign_slice(a, b):
    _chk(a, np.float32), _chk(b, np.float32)
    if lib().ora_add_assign_slice(_p(a), a.size, _p(b), b.size):
        raise OracleError("assert_eq!(a.len(), b.len())")


def add_assign_par(a, b, threads):
    _chk(a, np.float32), _chk(b, np.float32)
    if lib().ora_add_assign_par(_p(a), a.size, _p(b), b.size, threads):
        raise OracleError("assert_eq!(a.len(), b.len())")


def add_scaled_slice(dst, src, scale):
    _chk(dst, np.float32), _chk(src, np.float32)
    if lib().ora_add_scaled_slice(_p(dst), dst.size, _p(src), src.size, scale):
        raise OracleError("assert_eq!(dst.len(), src.len())")


def add_rmsnorm_rows(x, delta, h, gamma, eps):
    """OP-B on [rows, n] arrays (f32 or fp16 bit patterns as uint16), in place on x, h."""
    rows, n = x.shape
    _chk(gamma, np.float32)
    if x.dtype == np.float32:
        lib().ora_add_rmsnorm_rows(_p(x), _p(delta), _p(h), _p(gamma), n, rows, eps)
    else:
        _chk(x, np.uint16)
        lib().ora_add_rmsnorm_rows_f16(_p(x), _p(delta), _p(h), _p(gamma), n, rows, eps)


# ---- rope
def rope_inv_freq(head_dim, base):
    out = np.zeros(head_dim // 2, np.float32)
    lib().ora_rope_inv_freq(head_dim, base, _p(out))
    return out


def rope_sin_cos(pos, inv):
    _chk(inv, np.float32)
    out = np.zeros((inv.size, 2), np.float32)
    lib().ora_rope_sin_cos(int(pos), _p(inv), inv.size, _p(out))
    return out


def rope_table(positions, inv):
    """[len(positions), half, 2] = the session table rows for these positions."""
    return np.stack([rope_sin_cos(p, inv) for p in positions]) if len(positions) else np.zeros((0, inv.size, 2), np.float32)


def rope_neox_cached_from_array(x, table):
    _chk(x, np.float32), _chk(table, np.float32)
    if lib().ora_rope_neox_cached_from_array(_p(x), x.size, _p(table), table.shape[0]):
        raise OracleError("assert!(x.len() >= table.len() * 2)")


def rope_norm_cached_from_array(x, table):
    _chk(x, np.float32), _chk(table, np.float32)
    if lib().ora_rope_norm_cached_from_array(_p(x), x.size, _p(table), table.shape[0]):
        raise OracleError("assert!(x.len() >= table.len() * 2)")


def rope_neox(x, pos, base):
    _chk(x, np.float32)
    lib().ora_rope_neox(_p(x), x.size, int(pos), base)


def rope_norm(x, pos, base):
    _chk(x, np.float32)
    lib().ora_rope_norm(_p(x), x.size, int(pos), base)


def add_bias_rows(rows, bias):
    """add_bias_rows (model/loader.rs:519-523), f32 in place."""
    _chk(rows, np.float32)
    _chk(bias, np.float32)
    lib().ora_add_bias_rows(_p(rows), rows.size, _p(bias), bias.size)


def qknorm_rope_rows(q, k, n_q, n_kv, head_dim, qw, kw, rope_flat, eps, style=0, q_bias=None, k_bias=None):
    """OP-C: q [rows, n_q*hd], k [rows, n_kv*hd] in place; rope_flat [rows, half, 2];
    style 0 = NeoX pairs, 1 = adjacent (NORM) pairs.  q_bias / k_bias: add_bias_rows first (attention.rs:125-129);
    fp16 rows are then widened, biased and run through the f32 op, and rounded once."""
    rows = q.shape[0]
    half = rope_flat.shape[1]
    _chk(rope_flat, np.float32)
    if q_bias is not None or k_bias is not None:
        f16 = q.dtype != np.float32
        qf = f16_bits_to_f32(q) if f16 else q
        kf = f16_bits_to_f32(k) if f16 else k
        if q_bias is not None and qf.size:
            add_bias_rows(qf, q_bias)
        if k_bias is not None and kf.size:
            add_bias_rows(kf, k_bias)
        lib().ora_qknorm_rope_rows_style(_p(qf), _p(kf), rows, n_q, n_kv, head_dim, _p(qw), _p(kw), _p(rope_flat), half, eps, style)
        if f16:
            q[...] = f32_to_f16_bits(qf)
            k[...] = f32_to_f16_bits(kf)
        return
    if q.dtype == np.float32:
        lib().ora_qknorm_rope_rows_style(_p(q), _p(k), rows, n_q, n_kv, head_dim, _p(qw), _p(kw), _p(rope_flat), half, eps, style)
    else:
        _chk(q, np.uint16)
        lib().ora_qknorm_rope_rows_style_f16(_p(q), _p(k), rows, n_q, n_kv, head_dim, _p(qw), _p(kw), _p(rope_flat), half, eps, style)


# ---- activation
def silu(x):
    return float(lib().ora_silu(float(np.float32(x))))


def swiglu(gate, up):
    if gate.dtype == np.float32:
        _chk(up, np.float32)
        if lib().ora_swiglu(_p(gate), gate.size, _p(up), up.size):
            raise OracleError("assert_eq!(gate.len(), up.len())")
    else:
        _chk(gate, np.uint16), _chk(up, np.uint16)
        if gate.size != up.size:
            raise OracleError("assert_eq!(gate.len(), up.len())")
        lib().ora_swiglu_f16(_p(gate), _p(up), gate.size)


def gelu_tanh_mul(x, u):
    return float(lib().ora_gelu_tanh_mul(float(np.float32(x)), float(np.float32(u))))


def geglu_tanh(gate, up):
    """ops::geglu_tanh (activation.rs:44-51) in place into gate; uint16 arrays: the fp16 storage form."""
    if gate.dtype == np.float32:
        _chk(up, np.float32)
        if lib().ora_geglu_tanh(_p(gate), gate.size, _p(up), up.size):
            raise OracleError("assert_eq!(gate.len(), up.len())")
    else:
        _chk(gate, np.uint16), _chk(up, np.uint16)
        if gate.size != up.size:
            raise OracleError("assert_eq!(gate.len(), up.len())")
        lib().ora_geglu_tanh_f16(_p(gate), _p(up), gate.size)


def softmax(x):
    _chk(x, np.float32)
    lib().ora_softmax(_p(x), x.size)


def sigmoid(x):
    _chk(x, np.float32)
    lib().ora_sigmoid(_p(x), x.size)


# ---- router
SOFTMAX, SIGMOID = 0, 1


def route_gated(logits, k, gating=SOFTMAX, norm=True, scale=1.0, bias=None):
    _chk(logits, np.float32)
    kk = min(k, logits.size)
    ids = np.zeros(kk, np.uint32)
    w = np.zeros(kk, np.float32)
    lib().ora_route_gated(_p(logits), logits.size, k, gating, int(norm), scale, _p(bias), _p(ids), _p(w))
    return ids, w


def topk_by_logits(logits, k):
    _chk(logits, np.float32)
    ids = np.zeros(min(k, logits.size), np.uint32)
    lib().ora_topk_by_logits(_p(logits), logits.size, k, _p(ids))
    return ids


def route(probs, k):
    _chk(probs, np.float32)
    kk = min(k, probs.size)
    ids = np.zeros(kk, np.uint32)
    w = np.zeros(kk, np.float32)
    lib().ora_route(_p(probs), probs.size, k, _p(ids), _p(w))
    return ids, w


def route_rows(logits, k, gating=SOFTMAX, norm=True, scale=1.0, bias=None, threads=1):
    _chk(logits, np.float32)
    rows, n = logits.shape
    kk = min(k, n)
    ids = np.zeros((rows, kk), np.uint32)
    w = np.zeros((rows, kk), np.float32)
    lib().ora_route_rows(_p(logits), rows, n, k, gating, int(norm), scale, _p(bias), _p(ids), _p(w), threads)
    return ids, w


def moe_group(ids, w, n_expert):
    _chk(ids, np.uint32), _chk(w, np.float32)
    rows, k = ids.shape
    table = np.zeros((n_expert, 3), np.uint32)
    tok = np.zeros(rows * k, np.uint32)
    tok_off = np.zeros(rows + 1, np.uint32)
    hit_row = np.zeros(rows * k, np.uint32)
    hit_w = np.zeros(rows * k, np.float32)
    n_used = lib().ora_moe_group(_p(ids), _p(w), rows, k, n_expert, _p(table), _p(tok), _p(tok_off), _p(hit_row), _p(hit_w))
    return table[:n_used].copy(), tok, tok_off, hit_row, hit_w


def moe_shared_hits(tok_off, hit_row, hit_w, total_rows):
    """prefill.rs:621-635, :658-675: one more hit per token, (total_rows + token, 1.0), after its routed ones."""
    rows = tok_off.size - 1
    n = int(tok_off[-1]) + rows
    to, hr, hw = np.zeros(rows + 1, np.uint32), np.zeros(n, np.uint32), np.zeros(n, np.float32)
    lib().ora_moe_shared_hits(_p(tok_off), _p(hit_row), _p(hit_w), rows, total_rows, _p(to), _p(hr), _p(hw))
    return to, hr, hw


def gather_rows(src, tok):
    tok = np.ascontiguousarray(tok, dtype=np.uint32)
    dst = np.zeros((tok.size, src.shape[1]), src.dtype)
    if src.dtype == np.float32:
        lib().ora_gather_rows(_p(src), _p(tok), tok.size, src.shape[1], _p(dst))
    else:
        _chk(src, np.uint16)
        lib().ora_gather_rows_f16(_p(src), _p(tok), tok.size, src.shape[1], _p(dst))
    return dst


def kv_store_rows(k, v, pos, k_cache, v_cache):
    """KvCache::store_at per row: k, v [rows, kv_dim] (f32, or fp16 bits) into the u16 caches [capacity, kv_dim]."""
    pos = np.ascontiguousarray(pos, dtype=np.uint32)
    rows, kv_dim = k.shape
    _chk(k_cache, np.uint16), _chk(v_cache, np.uint16)
    fn = lib().ora_kv_store_rows if k.dtype == np.float32 else lib().ora_kv_store_rows_f16
    if fn(_p(k), _p(v), rows, kv_dim, _p(pos), k_cache.shape[0], _p(k_cache), _p(v_cache)):
        raise OracleError("position past capacity")


def moe_combine_add_rmsnorm(x, flat, tok_off, hit_row, hit_w, h, gamma, eps):
    """x [rows, n] += weighted hits of flat [total_rows, n]; h = rmsnorm(x) * gamma (h may be None)."""
    rows, n = x.shape
    _chk(tok_off, np.uint32), _chk(hit_row, np.uint32), _chk(hit_w, np.float32)
    fn = lib().ora_moe_combine_add_rmsnorm if x.dtype == np.float32 else lib().ora_moe_combine_add_rmsnorm_f16
    fn(_p(x), _p(flat), _p(tok_off), _p(hit_row), _p(hit_w), _p(h), _p(gamma), n, rows, eps)


def argmax_last(logits):
    _chk(logits, np.float32)
    return int(lib().ora_argmax_last(_p(logits), logits.size))

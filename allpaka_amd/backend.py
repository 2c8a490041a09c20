"""Host-side mirror of the reference's operator surface over the C ABI.

Names, argument meaning and error behaviour follow `allpaka_backend::ops`
(crates/allpaka-backend/src/ops/*.rs), `QuantMat` (quantmat/mod.rs:39-89) and
`model::route_gated` (crates/allpaka-model/src/model/moe.rs:601-616):
  * where the reference panics on a length mismatch, these raise AssertionError;
  * where the reference returns Err (QuantMat, dequant), these raise ValueError;
  * where an accelerator entry would decline (`None`), these raise `Declined`.
Tensors are torch CUDA tensors (float32, or float16 for the fp16 activation
form); every op runs in place where the reference's does.
"""
import ctypes as C
import contextlib
import enum

import torch

from . import lib as _l
from .lib import Declined, check  # noqa: F401


class Gating(enum.IntEnum):
    Softmax = 0
    Sigmoid = 1


class GgmlType(enum.IntEnum):
    """Values are the unified dequant format codes (gpu/common.rs:47-61)."""
    Q4K = 0
    Q5K = 1
    Q6K = 2
    Q8_0 = 3
    Q2K = 4
    Q3K = 5
    Q5_0 = 6
    F16 = 7
    F32 = 8
    BF16 = 9


def _dt(t):
    if t.dtype == torch.float32:
        return _l.F32
    if t.dtype == torch.float16:
        return _l.F16
    raise Declined(_l.DECLINE_UNSUPPORTED, f"activation dtype {t.dtype}")


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):  # a device address from Backend.resolve
        return t
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensors only"
    return t.data_ptr()


class Backend:
    """One device context (`apk_ctx`): the process-wide backend singleton of the
    reference (`with_gpu`, gpu/cuda/runtime/device.rs:944-948)."""

    def __init__(self, device=0):
        self.L = _l.load()
        h = C.c_void_p()
        check(self.L.apk_init(device, C.byref(h)))
        self.h = h
        self.device = torch.device("cuda", device)
        self._recording = False

    def close(self):
        if self.h:
            self.L.apk_shutdown(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- runtime
    def sync(self):
        check(self.L.apk_sync(self.h))

    def stats(self):
        v = [C.c_uint64() for _ in range(4)]
        check(self.L.apk_stats(self.h, *[C.byref(x) for x in v]))
        return tuple(x.value for x in v)

    def take_faults(self):
        f = C.c_uint32()
        check(self.L.apk_take_faults(self.h, C.byref(f)))
        return f.value

    # ---- ownership: gpu::attach / detach / resolve_w (gpu/stub.rs:37-41, gpu/cuda/runtime/select.rs:80-84)
    @staticmethod
    def _host_range(a):
        assert a.flags["C_CONTIGUOUS"], "a contiguous host array"
        return a.ctypes.data, a.nbytes

    def attach(self, mapping):
        """gpu::attach(mapping) -> bool: the host array's bytes are copied to the device once and keyed by host address;
        the same mapping again adds an owner, a range inside an attached one needs no copy."""
        p, n = self._host_range(mapping)
        rc = self.L.apk_attach(self.h, p, n)
        if rc < 0:
            check(rc)
        return rc == 0

    def detach(self, mapping):
        """gpu::detach(mapping) -> bool: drops one owner; False (and nothing else) when the mapping was not attached.
        The last owner frees the device copy; graphs recorded while the mapping was attached decline their replays
        from then on (they hold the old addresses), as the reference drops its own graphs there."""
        p, n = self._host_range(mapping)
        rc = self.L.apk_detach_range(self.h, p, n)
        if rc not in (0, _l.DECLINE_NOT_ATTACHED):
            check(rc)
        return rc == 0

    def owners(self, mapping):
        p, n = self._host_range(mapping)
        v = C.c_size_t()
        check(self.L.apk_attached_owners(self.h, p, n, C.byref(v)))
        return v.value

    def resolve(self, host_slice):
        """resolve_w: the device address of a host array inside an attached mapping, or None for foreign memory."""
        p, n = self._host_range(host_slice)
        dev = C.c_void_p()
        rc = self.L.apk_resolve(self.h, p, n, C.byref(dev))
        if rc == _l.DECLINE_NOT_ATTACHED:
            return None
        check(rc)
        return dev.value

    def _enter(self):
        # torch owns the buffers and fills them on its own stream
        torch.cuda.current_stream(self.device).synchronize()

    def _leave(self):
        # the mirrored ops return with their result in place, like the CPU ops they stand
        # for; inside a recording nothing runs, so there is nothing to wait for
        if not self._recording:
            self.sync()

    # ---- record / replay (stream capture of gpu/cuda/prefill.rs:52-108)
    def capture_begin(self):
        self._enter()
        check(self.L.apk_capture_begin(self.h))
        self._recording = True

    def capture_end(self):
        g = C.c_void_p()
        self._recording = False
        check(self.L.apk_capture_end(self.h, C.byref(g)))
        return Graph(self, g)

    def capture_abort(self):
        self._recording = False
        check(self.L.apk_capture_abort(self.h))

    @contextlib.contextmanager
    def record(self):
        """`with be.record() as rec: <ops>` -> `rec.graph` replays them with one submission."""
        rec = _Recording()
        self.capture_begin()
        try:
            yield rec
        except BaseException:
            self.capture_abort()
            raise
        rec.graph = self.capture_end()

    # ---- ops::* (crates/allpaka-backend/src/ops)
    def rmsnorm(self, x, weight, eps):
        """ops::rmsnorm (norm.rs:115): in place over ONE row."""
        assert x.numel() == weight.numel()
        self._rows(x, None, x, weight, weight.numel(), 1, eps)

    def rmsnorm_into(self, dst, src, weight, eps):
        """ops::rmsnorm_into (norm.rs:193)."""
        assert src.numel() == weight.numel()
        assert dst.numel() == src.numel()
        self._rows(src, None, dst, weight, weight.numel(), 1, eps)

    def rmsnorm_rows_into(self, dst, src, weight, eps):
        """ops::rmsnorm_rows_into (norm.rs:275): rows = src.len() / weight.len()."""
        n = weight.numel()
        rows = src.numel() // n
        assert dst.numel() >= rows * n, "dst holds fewer rows than src"
        self._enter()
        check(self.L.apk_add_rmsnorm_rows(self.h, _ptr(src), None, _ptr(dst), _ptr(weight), n, rows, eps, _dt(src)))
        self._leave()

    def add_assign_slice(self, a, b):
        """ops::add_assign_slice (blas.rs:105): a += b.  Where a norm follows, add_rmsnorm_rows
        does both in one pass."""
        assert a.numel() == b.numel()
        assert a.dtype == b.dtype
        self._enter()
        check(self.L.apk_add_assign(self.h, _ptr(a), _ptr(b), a.numel(), _dt(a)))
        self._leave()

    def add_scaled_slice(self, dst, src, scale):
        """ops::add_scaled_slice (blas.rs:25-102): dst = fma(src, scale, dst), the per-expert step of the decode MoE
        combine (moe.rs:500-509).  A whole batch's combine is moe_combine_add_rmsnorm."""
        assert dst.numel() == src.numel()
        assert dst.dtype == src.dtype
        self._enter()
        check(self.L.apk_add_scaled(self.h, _ptr(dst), _ptr(src), dst.numel(), float(scale), _dt(dst)))
        self._leave()

    def softmax(self, x):
        """ops::softmax (activation.rs:5) over each row of x (or over a 1-D x), in place."""
        assert x.dtype == torch.float32
        rows, n = (1, x.numel()) if x.dim() == 1 else (x.shape[0], x.shape[1])
        self._enter()
        check(self.L.apk_softmax_rows(self.h, _ptr(x), rows, n))
        self._leave()

    def add_rmsnorm_rows(self, x, delta, h, gamma, eps):
        """x += delta; h = rmsnorm(x) * gamma, rows = x.len() / gamma.len()
        (model/decode.rs:584 then :764, one launch)."""
        n = gamma.numel()
        assert x.numel() % n == 0
        rows = x.numel() // n
        if delta is not None:
            assert delta.numel() == x.numel()
            assert delta.dtype == x.dtype
        assert h.numel() >= rows * n, "dst holds fewer rows than src"
        assert h.dtype == x.dtype
        self._rows(x, delta, h, gamma, n, rows, eps)

    def postnorm_add_rmsnorm_rows(self, x, delta, post_gamma, h, gamma, eps):
        """The sandwich norm of the Gemma family and the next norm in one pass: x += rmsnorm(delta) * post_gamma
        (ops::rmsnorm on the projected rows, then add_assign_slice: decode.rs:581-584, :771-775), h = rmsnorm(x) * gamma.
        delta may be overwritten with its normalised form."""
        n = gamma.numel()
        rows = x.numel() // n
        assert x.numel() == rows * n == delta.numel() and h.numel() >= rows * n and post_gamma.numel() == n
        assert x.dtype == delta.dtype == h.dtype
        self._enter()
        check(self.L.apk_postnorm_add_rmsnorm_rows(self.h, _ptr(x), _ptr(delta), _ptr(post_gamma), _ptr(h), _ptr(gamma), n, rows, eps, _dt(x)))
        self._leave()

    def _rows(self, x, delta, h, gamma, n, rows, eps):
        assert gamma.dtype == torch.float32
        self._enter()
        check(self.L.apk_add_rmsnorm_rows(self.h, _ptr(x), _ptr(delta), _ptr(h), _ptr(gamma), n, rows, eps, _dt(x)))
        self._leave()

    def rope_inv_freq(self, rot_dim, base):
        """ops::rope_inv_freq (rope.rs:8-12): the f32 inverse frequencies, computed on the host, as a device tensor."""
        import numpy as np

        inv = np.empty(rot_dim // 2, np.float32)
        check(self.L.apk_rope_inv_freq(rot_dim, base, inv.ctypes.data))
        return torch.from_numpy(inv).to(self.device)

    def rope_table(self, positions, inv_freq):
        """ops::rope_sin_cos per position -> [rows, half, 2] = [sin, cos] (rope.rs:18-22)."""
        rows, half = positions.numel(), inv_freq.numel()
        assert positions.dtype in (torch.int32, torch.uint32) and inv_freq.dtype == torch.float32
        table = torch.empty((rows, half, 2), dtype=torch.float32, device=self.device)
        self._enter()
        check(self.L.apk_rope_table(self.h, _ptr(positions), _ptr(inv_freq), rows, half, _ptr(table)))
        self._leave()
        return table

    def rope_table_into(self, positions, inv_freq, table):
        """rope_table into a caller's [rows, half, 2] tensor: the form a recorded decode step uses
        (the positions live in a device buffer the caller rewrites between replays)."""
        rows, half = positions.numel(), inv_freq.numel()
        assert positions.dtype in (torch.int32, torch.uint32) and inv_freq.dtype == torch.float32
        assert table.dtype == torch.float32 and table.numel() == rows * half * 2
        self._enter()
        check(self.L.apk_rope_table(self.h, _ptr(positions), _ptr(inv_freq), rows, half, _ptr(table)))
        self._leave()

    def qknorm_rope_norm(self, q, k, q_norm, k_norm, rope_flat, n_q, n_kv, head_dim, eps, rot_dim=None):
        """The same loop for RopeStyle::Norm models: adjacent pairs (2i, 2i+1) rotate
        (rope_norm_cached_from_array, rope.rs:52-64; attention.rs:62-67)."""
        self.qknorm_rope_neox(q, k, q_norm, k_norm, rope_flat, n_q, n_kv, head_dim, eps, rot_dim, _entry="apk_qknorm_rope_norm")

    def rope_norm_cached_from_array(self, x, table):
        """ops::rope_norm_cached_from_array (rope.rs:52) on one head."""
        assert x.numel() >= table.shape[0] * 2
        self.qknorm_rope_norm(x, x[:0], None, None, table, 1, 0, x.numel(), 0.0, rot_dim=table.shape[0] * 2)

    def qknorm_rope_neox(self, q, k, q_norm, k_norm, rope_flat, n_q, n_kv, head_dim, eps, rot_dim=None,
                         _entry="apk_qknorm_rope_neox"):
        """The QK-norm + RoPE loop of run_cpu_attention_from_qkv (attention.rs:131-165):
        q [rows, n_q*head_dim], k [rows, n_kv*head_dim] in place; rope_flat [rows, half, 2]
        (half = rot_dim/2 <= head_dim/2: partial rotary leaves the tail of a head unrotated)."""
        rows = q.numel() // (n_q * head_dim) if n_q else k.numel() // (n_kv * head_dim)
        assert q.numel() == rows * n_q * head_dim and k.numel() == rows * n_kv * head_dim
        rot = head_dim if rot_dim is None else rot_dim
        assert rope_flat.dtype == torch.float32 and rope_flat.numel() == rows * (rot // 2) * 2
        assert q.dtype == k.dtype
        for w in (q_norm, k_norm):
            assert w is None or (w.numel() == head_dim and w.dtype == torch.float32)
        self._enter()
        check(getattr(self.L, _entry)(self.h, _ptr(q), _ptr(k), _ptr(q_norm), _ptr(k_norm), _ptr(rope_flat), rows,
                                      n_q, n_kv, head_dim, rot, eps, _dt(q)))
        self._leave()

    def qknorm_rope_kv_store(self, q, k, v, q_norm, k_norm, rope_flat, cache_pos, k_cache, v_cache, n_q, n_kv, head_dim, eps,
                             adjacent_pairs=False, rot_dim=None):
        """qknorm_rope_neox (adjacent_pairs: qknorm_rope_norm), then KvCache::store_at of every row's k and v as
        f16 at cache row cache_pos[r] (kv.rs:682-697), in one launch.  k_cache, v_cache: fp16 [capacity, n_kv*head_dim]."""
        rows = k.numel() // (n_kv * head_dim)
        assert q.numel() == rows * n_q * head_dim and v.numel() == k.numel() == rows * n_kv * head_dim
        rot_dim = head_dim if rot_dim is None else rot_dim
        assert rope_flat.numel() == rows * rot_dim and q.dtype == k.dtype == v.dtype
        assert k_cache.dtype == v_cache.dtype == torch.float16 and k_cache.shape == v_cache.shape
        assert k_cache.shape[1] == n_kv * head_dim and cache_pos.numel() == rows
        self._enter()
        fn = self.L.apk_qknorm_rope_norm_kv_store if adjacent_pairs else self.L.apk_qknorm_rope_kv_store
        check(fn(self.h, _ptr(q), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm), _ptr(rope_flat), _ptr(cache_pos), _ptr(k_cache),
                 _ptr(v_cache), k_cache.shape[0], rows, n_q, n_kv, head_dim, rot_dim, eps, _dt(q)))
        self._leave()
        # (inside a recording nothing has run yet: the caller reads take_faults() after a replay)
        if not self._recording and self.take_faults() & _l.FAULT_CACHE_RANGE:
            raise AssertionError("position past capacity")

    def qknorm_rope_pos(self, q, k, q_norm, k_norm, positions, inv_freq, n_q, n_kv, head_dim, eps, adjacent_pairs=False,
                        rot_dim=None, v=None, k_cache=None, v_cache=None):
        """The QK-norm + RoPE step of a decode-sized batch (at most 64 rows) with the angles taken from the rows' positions
        inside the launch: rope_sin_cos(pos, inv_freq) per row (rope.rs:18-22) instead of a table; with k_cache / v_cache
        (fp16 [capacity, n_kv*head_dim]) also KvCache::store_at at row positions[r] (kv.rs:682-697).  The reference's
        rmsnorm_rope_freq_dpos / rmsnorm_rope_store_freq_dpos (gpu/cuda/kernels.rs:577-671)."""
        rows = q.numel() // (n_q * head_dim) if n_q else k.numel() // (n_kv * head_dim)
        rot = head_dim if rot_dim is None else rot_dim
        assert q.numel() == rows * n_q * head_dim and k.numel() == rows * n_kv * head_dim and q.dtype == k.dtype
        assert positions.numel() == rows and positions.dtype == torch.int32
        assert inv_freq.dtype == torch.float32 and inv_freq.numel() == rot // 2
        cap = 0
        if k_cache is not None:
            assert v is not None and v.numel() == k.numel() and v.dtype == k.dtype and v_cache is not None
            assert k_cache.dtype == v_cache.dtype == torch.float16 and k_cache.shape == v_cache.shape and k_cache.shape[1] == n_kv * head_dim
            cap = k_cache.shape[0]
        self._enter()
        check(self.L.apk_qknorm_rope_pos(self.h, _ptr(q), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm), _ptr(positions), _ptr(inv_freq),
                                         _ptr(k_cache), _ptr(v_cache), cap, rows, n_q, n_kv, head_dim, rot, 1 if adjacent_pairs else 0, eps, _dt(q)))
        self._leave()
        if k_cache is not None and not self._recording and self.take_faults() & _l.FAULT_CACHE_RANGE:
            raise AssertionError("position past capacity")

    def cast(self, src, dtype):
        """allpaka_dtype::f32_to_f16 / f16_to_f32 over a tensor (dtype/src/lib.rs:129-184), bit for bit."""
        assert src.dtype in (torch.float32, torch.float16) and dtype in (torch.float32, torch.float16) and dtype != src.dtype
        dst = torch.empty(src.shape, dtype=dtype, device=self.device)
        self._enter()
        check(self.L.apk_cast(self.h, _ptr(src), _dt(src), _ptr(dst), _dt(dst), src.numel()))
        self._leave()
        return dst

    def add_bias_rows(self, x, bias):
        """add_bias_rows (model/loader.rs:519-523): x[r][i] += bias[i] over rows of bias.numel() elements."""
        n = bias.numel()
        assert n > 0 and x.numel() % n == 0 and bias.dtype == torch.float32
        self._enter()
        check(self.L.apk_add_bias_rows(self.h, _ptr(x), _ptr(bias), x.numel() // n, n, _dt(x)))
        self._leave()

    def attn_prologue_args(self, q, k, v, n_q, n_kv, head_dim, eps, rope_flat, q_bias=None, k_bias=None, v_bias=None, q_norm=None,
                           k_norm=None, cache_pos=None, k_cache=None, v_cache=None, adjacent_pairs=False, rot_dim=None):
        """The struct apk_attn_prologue for these tensors (kept alive by the caller)."""
        rows = q.numel() // (n_q * head_dim) if n_q else k.numel() // (n_kv * head_dim)
        rot_dim = head_dim if rot_dim is None else rot_dim
        assert q.numel() == rows * n_q * head_dim and k.numel() == rows * n_kv * head_dim and rope_flat.numel() == rows * rot_dim
        assert v is None or (v.numel() == k.numel() and v.dtype == k.dtype)
        for b, heads in ((q_bias, n_q), (k_bias, n_kv), (v_bias, n_kv)):
            assert b is None or (b.dtype == torch.float32 and b.numel() == heads * head_dim)
        if k_cache is not None:
            assert k_cache.dtype == v_cache.dtype == torch.float16 and k_cache.shape == v_cache.shape
            assert k_cache.shape[1] == n_kv * head_dim and cache_pos.numel() == rows
        a = _l.AttnPrologue()
        a.q, a.k, a.v = _ptr(q), _ptr(k), _ptr(v)
        a.q_bias, a.k_bias, a.v_bias = _ptr(q_bias), _ptr(k_bias), _ptr(v_bias)
        a.q_norm, a.k_norm, a.rope = _ptr(q_norm), _ptr(k_norm), _ptr(rope_flat)
        a.cache_pos, a.k_cache, a.v_cache = _ptr(cache_pos), _ptr(k_cache), _ptr(v_cache)
        a.capacity = 0 if k_cache is None else k_cache.shape[0]
        a.rows, a.n_q, a.n_kv, a.head_dim, a.rot_dim = rows, n_q, n_kv, head_dim, rot_dim
        a.eps, a.dtype, a.adjacent_pairs = eps, _dt(q), int(adjacent_pairs)
        return a

    def attn_prologue_rows(self, q, k, v, n_q, n_kv, head_dim, eps, rope_flat, **kw):
        """The q/k/v rows between the QKV projection and attention (attention.rs:125-165, kv.rs:682-697): optional
        projection biases, optional per-head norms, the rotation, and the optional K/V cache store, as one call."""
        a = self.attn_prologue_args(q, k, v, n_q, n_kv, head_dim, eps, rope_flat, **kw)
        self._enter()
        check(self.L.apk_attn_prologue_rows(self.h, C.byref(a)))
        self._leave()
        if kw.get("k_cache") is not None and not self._recording and self.take_faults() & _l.FAULT_CACHE_RANGE:
            raise AssertionError("position past capacity")

    def layer_prologue(self, x, delta, h, gamma, q, k, q_norm, k_norm, rope_flat, n_q, n_kv, head_dim, eps):
        """add_rmsnorm_rows(x, delta, h, gamma) and qknorm_rope_neox(q, k, ...) as one launch
        (small decode batches; larger ones run as the two launches)."""
        n = gamma.numel()
        rows = x.numel() // n
        assert x.numel() == rows * n and h.numel() >= rows * n and (delta is None or delta.numel() == x.numel())
        assert q.numel() == rows * n_q * head_dim and k.numel() == rows * n_kv * head_dim
        assert rope_flat.numel() == rows * head_dim and q.dtype == k.dtype == x.dtype
        self._enter()
        check(self.L.apk_layer_prologue(self.h, _ptr(x), _ptr(delta), _ptr(h), _ptr(gamma), n, _ptr(q), _ptr(k), _ptr(q_norm),
                                        _ptr(k_norm), _ptr(rope_flat), rows, n_q, n_kv, head_dim, head_dim, eps, _dt(x)))
        self._leave()

    def rope_neox_cached_from_array(self, x, table):
        """ops::rope_neox_cached_from_array (rope.rs:70) on one head."""
        assert x.numel() >= table.shape[0] * 2
        self.qknorm_rope_neox(x, x[:0], None, None, table, 1, 0, x.numel(), 0.0, rot_dim=table.shape[0] * 2)

    def swiglu(self, gate, up):
        """ops::swiglu (activation.rs:57): gate = silu(gate) * up."""
        assert gate.numel() == up.numel()
        assert gate.dtype == up.dtype
        self._enter()
        check(self.L.apk_swiglu(self.h, _ptr(gate), _ptr(up), gate.numel(), _dt(gate)))
        self._leave()

    def geglu_tanh(self, gate, up):
        """ops::geglu_tanh (activation.rs:44-51): gate = gelu_tanh(gate) * up, the Gemma-family FFN gate."""
        assert gate.numel() == up.numel()
        assert gate.dtype == up.dtype
        self._enter()
        check(self.L.apk_geglu_tanh(self.h, _ptr(gate), _ptr(up), gate.numel(), _dt(gate)))
        self._leave()

    # ---- model::route_gated (crates/allpaka-model/src/model/moe.rs:601)
    def route_rows(self, logits, k, gating=Gating.Softmax, norm=True, scale=1.0, bias=None):
        """route_gated_into_slice for every row of logits [rows, n_expert] -> (ids u32, w f32) [rows, k]."""
        rows, n = logits.shape
        k = min(k, n)
        ids = torch.empty((rows, k), dtype=torch.int32, device=self.device)
        w = torch.empty((rows, k), dtype=torch.float32, device=self.device)
        if k == 0:
            return ids, w
        assert logits.dtype == torch.float32
        self._enter()
        check(self.L.apk_route_topk(self.h, _ptr(logits), _ptr(bias), rows, n, k, int(norm), scale,
                                    int(gating == Gating.Sigmoid), _ptr(ids), _ptr(w)))
        self._leave()
        return ids, w

    def route(self, probs, k):
        """model::route(probs, k) (moe.rs:623-658): the top k of an already softmaxed row, renormalised -> list of
        (expert, weight), best first."""
        n = probs.numel()
        k = min(k, n)
        if k == 0:
            return []
        ids = torch.empty((1, k), dtype=torch.int32, device=self.device)
        w = torch.empty((1, k), dtype=torch.float32, device=self.device)
        self._enter()
        check(self.L.apk_route_topk(self.h, _ptr(probs), None, 1, n, k, 1, 1.0, 2, _ptr(ids), _ptr(w)))
        self._leave()
        return list(zip(ids[0].tolist(), w[0].tolist()))

    def route_gated(self, logits, k, gating=Gating.Softmax, norm=True, scale=1.0, bias=None):
        """model::route_gated on one row -> list of (expert, weight), best first."""
        ids, w = self.route_rows(logits.reshape(1, -1), k, gating, norm, scale, bias)
        return list(zip(ids[0].tolist(), w[0].tolist()))

    def moe_permute(self, ids, w, n_expert):
        """groups/used/table/tok + CSR of Ffn::moe_batch (moe.rs:229-271, prefill.rs:624-675)."""
        rows, k = ids.shape
        dev = self.device
        table = torch.zeros((n_expert, 3), dtype=torch.int32, device=dev)
        n_used = torch.zeros(1, dtype=torch.int32, device=dev)
        tok = torch.empty(rows * k, dtype=torch.int32, device=dev)
        tok_off = torch.empty(rows + 1, dtype=torch.int32, device=dev)
        hit_row = torch.empty(rows * k, dtype=torch.int32, device=dev)
        hit_w = torch.empty(rows * k, dtype=torch.float32, device=dev)
        self._enter()
        check(self.L.apk_moe_permute(self.h, _ptr(ids), _ptr(w), rows, k, n_expert, _ptr(table), _ptr(n_used), _ptr(tok),
                                     _ptr(tok_off), _ptr(hit_row), _ptr(hit_w)))
        self._leave()
        if self._recording:  # nothing has run: the whole table, of which a replay fills the leading rows
            return table, tok, tok_off, hit_row, hit_w
        return table[: int(n_used.item())], tok, tok_off, hit_row, hit_w

    def moe_shared_hits(self, tok_off, hit_row, hit_w, total_rows):
        """The shared expert's hit per token (prefill.rs:621-635): (total_rows + token, 1.0) after the routed hits.
        Returns the lengthened (tok_off, hit_row, hit_w)."""
        rows = tok_off.numel() - 1
        n = hit_row.numel() + rows
        dev = self.device
        to = torch.empty(rows + 1, dtype=torch.int32, device=dev)
        hr = torch.empty(n, dtype=torch.int32, device=dev)
        hw = torch.empty(n, dtype=torch.float32, device=dev)
        self._enter()
        check(self.L.apk_moe_shared_hits(self.h, _ptr(tok_off), _ptr(hit_row), _ptr(hit_w), rows, total_rows, _ptr(to), _ptr(hr), _ptr(hw)))
        self._leave()
        return to, hr, hw

    def route_group(self, logits, k, n_expert=None, gating=Gating.Softmax, norm=True, scale=1.0, bias=None):
        """route_rows then moe_permute with the same results; one launch for a decode-sized batch
        (the router and the grouping of Ffn::moe_batch, moe.rs:204-271, :298-309).
        Returns (ids, w), (table, tok, tok_off, hit_row, hit_w)."""
        rows, n = logits.shape
        n_expert = n if n_expert is None else n_expert
        k = min(k, n)
        dev = self.device
        assert logits.dtype == torch.float32 and n_expert == n
        ids = torch.empty((rows, k), dtype=torch.int32, device=dev)
        w = torch.empty((rows, k), dtype=torch.float32, device=dev)
        table = torch.zeros((n_expert, 3), dtype=torch.int32, device=dev)
        n_used = torch.zeros(1, dtype=torch.int32, device=dev)
        tok = torch.empty(rows * k, dtype=torch.int32, device=dev)
        tok_off = torch.empty(rows + 1, dtype=torch.int32, device=dev)
        hit_row = torch.empty(rows * k, dtype=torch.int32, device=dev)
        hit_w = torch.empty(rows * k, dtype=torch.float32, device=dev)
        self._enter()
        check(self.L.apk_route_group(self.h, _ptr(logits), _ptr(bias), rows, n_expert, k, int(norm), scale,
                                     int(gating == Gating.Sigmoid), _ptr(ids), _ptr(w), _ptr(table), _ptr(n_used), _ptr(tok),
                                     _ptr(tok_off), _ptr(hit_row), _ptr(hit_w)))
        self._leave()
        if self._recording:
            return (ids, w), (table, tok, tok_off, hit_row, hit_w)
        return (ids, w), (table[: int(n_used.item())], tok, tok_off, hit_row, hit_w)

    def gather_rows(self, src, tok):
        """xe rows in tok order (moe.rs:348-352)."""
        total = tok.numel()
        dst = torch.empty((total, src.shape[1]), dtype=src.dtype, device=self.device)
        self._enter()
        check(self.L.apk_gather_rows(self.h, _ptr(src), _ptr(tok), src.shape[0], total, src.shape[1], _ptr(dst), _dt(src)))
        self._leave()
        return dst

    def scatter_rows(self, src, hit_row, k):
        """The same xe rows from the token side: xe[hit_row[t*k+j]] = src[t] (each row read once)."""
        rows = src.shape[0]
        total = rows * k
        dst = torch.empty((total, src.shape[1]), dtype=src.dtype, device=self.device)
        self._enter()
        check(self.L.apk_scatter_rows(self.h, _ptr(src), _ptr(hit_row), rows, k, total, src.shape[1], _ptr(dst), _dt(src)))
        self._leave()
        return dst

    def moe_combine_add_rmsnorm(self, x, flat, tok_off, hit_row, hit_w, h, gamma, eps):
        """x[t] += sum over the token's hits of hit_w * flat[hit_row] (add_scaled_slice order), then
        h = rmsnorm(x) * gamma (moe.rs:298-333 + the residual add + the next norm); h=None: no norm.
        tok_off=None: every token has flat.shape[0] / rows hits (no shared expert), token t's at [t*k, (t+1)*k)."""
        n = flat.shape[1]
        rows = x.numel() // n
        assert x.numel() == rows * n and (tok_off is None or tok_off.numel() == rows + 1) and flat.dtype == x.dtype
        assert h is None or (h.numel() >= rows * n and gamma is not None and gamma.numel() == n)
        self._enter()
        check(self.L.apk_moe_combine_add_rmsnorm(self.h, _ptr(x), _ptr(flat), _ptr(tok_off), _ptr(hit_row), _ptr(hit_w),
                                                 flat.shape[0], _ptr(h), _ptr(gamma), n, rows, eps, _dt(x)))
        self._leave()

    def argmax_rows(self, logits):
        """Greedy pick per row: (0..n).max_by(total_cmp) of forward_greedy (decode.rs:628-630)."""
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
        self.argmax_rows_into(logits, out)
        self._leave()
        return out

    def argmax_rows_into(self, logits, out):
        """The same into a caller's int32 tensor, enqueued only (no wait)."""
        rows, n = logits.shape
        assert logits.dtype == torch.float32 and out.dtype == torch.int32 and out.numel() >= rows
        self._enter()
        check(self.L.apk_argmax_rows(self.h, _ptr(logits), rows, n, _ptr(out)))


class _Recording:
    graph = None


class Graph:
    """A recorded chain of ops (`apk_graph`); every pointer and size is baked in, so the
    tensors the ops were recorded with must stay alive and in place."""

    def __init__(self, backend, handle):
        self.be, self.g = backend, handle

    @property
    def nodes(self):
        n = C.c_size_t()
        check(self.be.L.apk_graph_nodes(self.g, C.byref(n)))
        return n.value

    def launch(self):
        check(self.be.L.apk_graph_launch(self.be.h, self.g))

    def destroy(self):
        if self.g:
            check(self.be.L.apk_graph_destroy(self.be.h, self.g))
            self.g = None


class QuantMat:
    """QuantMat::{new,row,row_into} (quantmat/mod.rs:39-89) over a device-resident table."""

    def __init__(self, backend, data, ty, n_out, n_in):
        ty = int(ty)
        rb = backend.L.apk_row_bytes(ty, n_in)
        if ty < 0 or ty > 9:
            raise ValueError(f"unsupported ggml type {ty}")
        if rb == 0:
            raise ValueError(f"row length {n_in} is not a whole number of blocks")
        if rb * n_out != data.numel() * data.element_size():
            raise ValueError(f"{n_out}x{n_in} needs {rb * n_out} bytes, got {data.numel() * data.element_size()}")
        self.b, self.data, self.ty, self.n_out, self.n_in, self.row_bytes = backend, data, ty, n_out, n_in, rb
        self.host = None

    @classmethod
    def from_mapping(cls, backend, host_bytes, ty, n_out, n_in):
        """QuantMat::new over a borrowed slice of an attached mapping (`data: &'a [u8]`, quantmat/mod.rs:39-66): the
        table is used where attach put it, named by its host address, and the address is resolved again at every call
        (resolve_w, gpu/cuda/runtime/select.rs:80-84) -- the QuantMat takes no owner, so once the mapping is detached
        every call raises Declined and launches nothing.  Foreign memory raises Declined, as the reference's
        accelerator declines it (its caller then runs the CPU path)."""
        ty = int(ty)
        rb = backend.L.apk_row_bytes(ty, n_in)
        if ty < 0 or ty > 9:
            raise ValueError(f"unsupported ggml type {ty}")
        if rb == 0:
            raise ValueError(f"row length {n_in} is not a whole number of blocks")
        if rb * n_out != host_bytes.nbytes:
            raise ValueError(f"{n_out}x{n_in} needs {rb * n_out} bytes, got {host_bytes.nbytes}")
        dev = backend.resolve(host_bytes)
        if dev is None:
            raise Declined(_l.DECLINE_NOT_ATTACHED, "the table is not inside an attached mapping")
        self = cls.__new__(cls)
        self.b, self.data, self.ty, self.n_out, self.n_in, self.row_bytes = backend, None, ty, n_out, n_in, rb
        self.host = host_bytes
        return self

    def _table(self):
        """the table's device address for this call"""
        if self.host is None:
            return _ptr(self.data)
        dev = self.b.resolve(self.host)
        if dev is None:
            raise Declined(_l.DECLINE_NOT_ATTACHED, "the table's mapping is no longer attached")
        return dev

    def row(self, j, dtype=torch.float32):
        out = torch.empty(self.n_in, dtype=dtype, device=self.b.device)
        self.row_into(j, out)
        return out

    def row_into(self, j, dst):
        if j >= self.n_out or j < 0:
            raise ValueError(f"row {j} out of {self.n_out}")
        if dst.numel() != self.n_in:
            raise ValueError(f"row_into destination has {dst.numel()} elements, expected {self.n_in}")
        ids = (C.c_uint32 * 1)(j)
        self.b._enter()
        check(self.b.L.apk_embed_rows_host_ids(self.b.h, self.ty, self._table(), self.n_out, self.n_in, ids, 1, _ptr(dst), _dt(dst)))
        self.b.sync()

    def dequant_rows(self, row0, count, dtype=torch.float16):
        """Rows [row0, row0 + count) dequantized without an id list: QuantMat::row_into over a range, or the
        reference's dequant_rows_f16 ahead of a dense GEMM (gpu/cuda/runtime/gemm.rs:213-260)."""
        out = torch.empty((count, self.n_in), dtype=dtype, device=self.b.device)
        self.b._enter()
        check(self.b.L.apk_dequant_rows(self.b.h, self.ty, self._table(), self.n_out, self.n_in, row0, count, _ptr(out), _dt(out)))
        self.b._leave()
        return out

    def rows_into(self, ids, dst, embed_scale=1.0):
        """The embedding loop of forward_batch (prefill.rs:92-109) as one launch; ids on the device;
        embed_scale: the multiplier of models that scale their token embeddings."""
        t = ids.numel()
        if dst.numel() != t * self.n_in:
            raise ValueError("destination size")
        self.b._enter()
        if embed_scale == 1.0:
            check(self.b.L.apk_embed_rows(self.b.h, self.ty, self._table(), self.n_out, self.n_in, _ptr(ids), t, _ptr(dst), _dt(dst)))
        else:
            check(self.b.L.apk_embed_rows_scaled(self.b.h, self.ty, self._table(), self.n_out, self.n_in, _ptr(ids), t,
                                                 embed_scale, _ptr(dst), _dt(dst)))
        self.b.sync()
        if self.b.take_faults() & _l.FAULT_TOKEN_RANGE:
            raise ValueError("token id out of vocab")


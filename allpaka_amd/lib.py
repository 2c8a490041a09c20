"""ctypes binding of libapk_hip.so (include/apk_hip.h).  Fails loudly when the
library has not been built: there is no fallback path."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libapk_hip.so")

F32, F16 = 0, 1
FMT_Q4K, FMT_Q5K, FMT_Q6K, FMT_Q8_0, FMT_Q2K, FMT_Q3K, FMT_Q5_0, FMT_F16, FMT_F32, FMT_BF16 = range(10)
DECLINE_UNSUPPORTED, DECLINE_SHAPE, DECLINE_NULL, DECLINE_RANGE, DECLINE_NO_DEVICE, DECLINE_NOT_ATTACHED, DECLINE_CAPTURE = range(1, 8)
FAULT_TOKEN_RANGE, FAULT_EXPERT_RANGE, FAULT_ROW_RANGE, FAULT_CACHE_RANGE = 1, 2, 4, 8



class Plan(C.Structure):
    """struct apk_plan: the kernel, grid and workgroup size an entry launches for a shape."""
    _fields_ = [("kernel", C.c_char * 64), ("grid", C.c_uint), ("block", C.c_uint), ("shmem", C.c_uint), ("variant", C.c_uint),
                ("tiles_per_lane", C.c_uint), ("waves_per_row", C.c_uint), ("rows_per_block", C.c_uint), ("lanes_per_row", C.c_uint),
                ("slices_per_row", C.c_uint), ("items", C.c_uint)]


class AttnPrologue(C.Structure):
    """struct apk_attn_prologue: the arguments of apk_attn_prologue_rows."""
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("q_bias", C.c_void_p), ("k_bias", C.c_void_p),
                ("v_bias", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p), ("rope", C.c_void_p),
                ("cache_pos", C.c_void_p), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p), ("capacity", C.c_size_t),
                ("rows", C.c_size_t), ("n_q", C.c_size_t), ("n_kv", C.c_size_t), ("head_dim", C.c_size_t), ("rot_dim", C.c_size_t),
                ("eps", C.c_float), ("dtype", C.c_int), ("adjacent_pairs", C.c_int)]


# every symbol include/apk_hip.h declares: (restype, argtypes)
_vp, _sz, _i, _f, _u64p, _u32p = C.c_void_p, C.c_size_t, C.c_int, C.c_float, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32)
_plan = C.POINTER(Plan)
SYMBOLS = {
    "apk_init": (_i, [_i, C.POINTER(_vp)]),
    "apk_shutdown": (_i, [_vp]),
    "apk_sync": (_i, [_vp]),
    "apk_stream": (_vp, [_vp]),
    "apk_last_error": (C.c_char_p, []),
    "apk_stats": (_i, [_vp, _u64p, _u64p, _u64p, _u64p]),
    "apk_take_faults": (_i, [_vp, _u32p]),
    "apk_row_bytes": (_sz, [_i, _sz]),
    "apk_can_embed": (_i, [_i, _sz]),
    "apk_malloc": (_i, [_vp, _sz, C.POINTER(_vp)]),
    "apk_free": (_i, [_vp, _vp]),
    "apk_h2d": (_i, [_vp, _vp, _vp, _sz]),
    "apk_d2h": (_i, [_vp, _vp, _vp, _sz]),
    "apk_attach": (_i, [_vp, _vp, _sz]),
    "apk_detach": (_i, [_vp, _vp]),
    "apk_detach_range": (_i, [_vp, _vp, _sz]),
    "apk_attached_owners": (_i, [_vp, _vp, _sz, C.POINTER(_sz)]),
    "apk_resolve": (_i, [_vp, _vp, _sz, C.POINTER(_vp)]),
    "apk_timer_begin": (_i, [_vp]),
    "apk_timer_end": (_i, [_vp, C.POINTER(_f)]),
    "apk_capture_begin": (_i, [_vp]),
    "apk_capture_end": (_i, [_vp, C.POINTER(_vp)]),
    "apk_capture_abort": (_i, [_vp]),
    "apk_graph_launch": (_i, [_vp, _vp]),
    "apk_graph_nodes": (_i, [_vp, C.POINTER(_sz)]),
    "apk_graph_destroy": (_i, [_vp, _vp]),
    "apk_embed_rows": (_i, [_vp, _i, _vp, _sz, _sz, _vp, _sz, _vp, _i]),
    "apk_embed_rows_scaled": (_i, [_vp, _i, _vp, _sz, _sz, _vp, _sz, _f, _vp, _i]),
    "apk_dequant_rows": (_i, [_vp, _i, _vp, _sz, _sz, _sz, _sz, _vp, _i]),
    "apk_embed_rows_host_ids": (_i, [_vp, _i, _vp, _sz, _sz, _vp, _sz, _vp, _i]),
    "apk_add_assign": (_i, [_vp, _vp, _vp, _sz, _i]),
    "apk_add_scaled": (_i, [_vp, _vp, _vp, _sz, _f, _i]),
    "apk_softmax_rows": (_i, [_vp, _vp, _sz, _sz]),
    "apk_add_rmsnorm_rows": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _f, _i]),
    "apk_qknorm_rope_neox": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _f, _i]),
    "apk_qknorm_rope_norm": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _f, _i]),
    "apk_qknorm_rope_kv_store": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _f, _i]),
    "apk_qknorm_rope_pos": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _i, _f, _i]),
    "apk_qknorm_rope_norm_kv_store": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _f, _i]),
    "apk_layer_prologue": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _f, _i]),
    "apk_rope_table": (_i, [_vp, _vp, _vp, _sz, _sz, _vp]),
    "apk_swiglu": (_i, [_vp, _vp, _vp, _sz, _i]),
    "apk_geglu_tanh": (_i, [_vp, _vp, _vp, _sz, _i]),
    "apk_route_topk": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _i, _f, _i, _vp, _vp]),
    "apk_moe_permute": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp, _vp]),
    "apk_gather_rows": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _vp, _i]),
    "apk_scatter_rows": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp, _i]),
    "apk_moe_combine_add_rmsnorm": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _sz, _sz, _f, _i]),
    "apk_argmax_rows": (_i, [_vp, _vp, _sz, _sz, _vp]),
    "apk_argmax_rows_noalloc": (_i, [_vp, _vp, _sz, _sz, _vp]),
    "apk_copy": (_i, [_vp, _vp, _vp, _sz]),
    "apk_rope_inv_freq": (_i, [_sz, _f, _vp]),
    "apk_route_group": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _i, _f, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "apk_plan_add_rmsnorm_rows": (_i, [_sz, _sz, _i, _plan]),
    "apk_plan_postnorm_add_rmsnorm_rows": (_i, [_sz, _sz, _i, _plan]),
    "apk_postnorm_add_rmsnorm_rows": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _f, _i]),
    "apk_plan_qknorm_rope": (_i, [_sz, _sz, _sz, _sz, _sz, _i, _i, _i, _plan]),
    "apk_plan_scatter_rows": (_i, [_sz, _sz, _sz, _i, _plan]),
    "apk_plan_attn_prologue_rows": (_i, [C.POINTER(AttnPrologue), _plan]),
    "apk_add_bias_rows": (_i, [_vp, _vp, _vp, _sz, _sz, _i]),
    "apk_cast": (_i, [_vp, _vp, _i, _vp, _i, _sz]),
    "apk_moe_shared_hits": (_i, [_vp, _vp, _vp, _vp, _sz, _sz, _vp, _vp, _vp]),
    "apk_attn_prologue_rows": (_i, [_vp, C.POINTER(AttnPrologue)]),
    "apk_plan_embed_rows": (_i, [_i, _sz, _sz, _i, _plan]),
    "apk_kernel_count": (_sz, []),
    "apk_kernel_name": (_i, [_sz, C.c_char_p, _sz]),
}


class ApkError(RuntimeError):
    """A HIP runtime failure (negative status)."""


class Declined(RuntimeError):
    """The device path declined the request (positive status): the reference's
    `None` / `AccelOutcome::Declined`.  `.reason` is the apk_decline code."""

    def __init__(self, reason, msg):
        super().__init__(f"declined({reason}): {msg}")
        self.reason = reason


def lib_path():
    return _SO


_lib = None


def load():
    """Loads the built library; raises if it is missing (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise ImportError(
                f"{_SO} is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
                "(or make -C allpaka_amd/csrc). allpaka_amd has no CPU fallback.")
        L = C.CDLL(_SO)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status):
    if status == 0:
        return
    msg = load().apk_last_error().decode(errors="replace")
    if status > 0:
        raise Declined(status, msg)
    raise ApkError(f"HIP error {-status}: {msg}")

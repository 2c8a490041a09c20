"""No-GPU checks of the boundary: the C-ABI library loads, exports every symbol
include/apk_hip.h declares, embeds a gfx950 code object, and its pure host
entries (block geometry, declines without a device) behave as the reference's
(crates/allpaka-backend/src/gpu/common.rs:102-153, gpu/stub.rs)."""
import ctypes as C
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    import allpaka_amd.lib as lib

    if not os.path.exists(lib.lib_path()):
        subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "allpaka_amd", "csrc")])
    return lib, lib.load()


def test_library_exports_every_declared_symbol():
    lib, L = _lib()
    header = open(os.path.join(ROOT, "include", "apk_hip.h")).read()
    declared = set(re.findall(r"\b(apk_[a-z0-9_]+)\s*\(", header))
    declared -= {"apk_ctx"}
    assert declared, "no declarations parsed"
    assert declared == set(lib.SYMBOLS), declared ^ set(lib.SYMBOLS)
    for name in declared:
        assert hasattr(L, name), name


def test_code_object_is_gfx950_and_embedded():
    lib, L = _lib()
    co = os.path.join(ROOT, "allpaka_amd", "csrc", "apk_kernels.hsaco")
    blob = open(lib.lib_path(), "rb").read()
    assert b"\x7fELF" in blob
    if os.path.exists(co):
        code = open(co, "rb").read()
        # hipcc --genco emits a clang offload bundle wrapping the gfx950 ELF; hipModuleLoadData takes both
        assert code[:4] in (b"\x7fELF", b"__CL") and code in blob, "code object is not embedded verbatim"
    assert b"gfx950" in blob
    for k in [b"apk_swiglu_f16", b"apk_add_rmsnorm_f16_c1", b"apk_qknorm_rope_f16_hd128", b"apk_embed_q4k_f16",
              b"apk_embed_q8_0_f32", b"apk_route_topk", b"apk_moe_permute", b"apk_gather_rows"]:
        assert k in blob, k


def test_row_bytes_and_format_codes_follow_the_reference():
    lib, L = _lib()
    # gpu/common.rs:106-115
    assert L.apk_row_bytes(lib.FMT_Q4K, 512) == 2 * 144
    assert L.apk_row_bytes(lib.FMT_Q6K, 256) == 210
    assert L.apk_row_bytes(lib.FMT_Q8_0, 64) == 2 * 34
    assert L.apk_row_bytes(lib.FMT_F16, 10) == 20
    assert L.apk_row_bytes(lib.FMT_F32, 3) == 12
    assert L.apk_row_bytes(lib.FMT_Q4K, 100) == 0
    assert L.apk_row_bytes(77, 256) == 0
    assert L.apk_row_bytes(lib.FMT_Q4K, 128) == 0
    assert L.apk_row_bytes(lib.FMT_Q5_0, 128) == 88
    # gpu/common.rs:118-134: the ten codes
    assert [lib.FMT_Q4K, lib.FMT_Q5K, lib.FMT_Q6K, lib.FMT_Q8_0, lib.FMT_Q2K, lib.FMT_Q3K, lib.FMT_Q5_0, lib.FMT_F16,
            lib.FMT_F32, lib.FMT_BF16] == list(range(10))
    assert L.apk_can_embed(lib.FMT_Q8_0, 1024) == 1 and L.apk_can_embed(lib.FMT_Q4K, 5120) == 1
    assert L.apk_can_embed(lib.FMT_Q4K, 100) == 0 and L.apk_can_embed(77, 256) == 0 and L.apk_can_embed(lib.FMT_F32, 3) == 0
    assert all(L.apk_can_embed(f, 512) == 1 for f in range(10))  # gpu_parity.rs:1147: all ten formats embed


def test_no_device_declines_instead_of_failing():
    lib, L = _lib()
    h = C.c_void_p()
    env_before = os.environ.get("ALLPAKA_NO_GPU")
    os.environ["ALLPAKA_NO_GPU"] = "1"  # capability.rs:58-61: the host can force the CPU path
    try:
        rc = L.apk_init(0, C.byref(h))
    finally:
        if env_before is None:
            del os.environ["ALLPAKA_NO_GPU"]
        else:
            os.environ["ALLPAKA_NO_GPU"] = env_before
    assert rc == lib.DECLINE_NO_DEVICE and not h.value
    assert b"ALLPAKA_NO_GPU" in L.apk_last_error()
    # NULL context: a decline status, never a crash
    assert L.apk_swiglu(None, None, None, 16, 0) == lib.DECLINE_NULL
    assert L.apk_sync(None) == lib.DECLINE_NULL


def test_package_has_no_cpu_fallback_and_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "allpaka_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h", ".S")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.lower().replace("no oracle", ""), f"{f} mentions the oracle"


def test_rope_inv_freq_is_the_reference_powf_series():
    """ops::rope_inv_freq (ops/rope.rs:8-12) on the host: base^(-2i/d) in f32 with libm's powf, the oracle's
    series bit for bit; the reference's own checks: inv[0] == 1, strictly decreasing (ops/mod.rs:250-257)."""
    import numpy as np

    import oracle as ora

    lib, L = _lib()
    for d, base in ((128, 1e6), (64, 1e4), (256, 1e6), (96, 5e5), (2, 10.0)):
        inv = np.zeros(d // 2, np.float32)
        assert L.apk_rope_inv_freq(d, base, inv.ctypes.data) == 0
        assert np.array_equal(inv.view(np.uint32), ora.rope_inv_freq(d, base).view(np.uint32))
        assert inv[0] == 1.0 and np.all(np.diff(inv) < 0)
    assert L.apk_rope_inv_freq(0, 1e4, None) == 0 and L.apk_rope_inv_freq(8, 1e4, None) == 3


def test_header_is_plain_c_and_the_ctypes_structs_have_its_layout(tmp_path):
    """include/apk_hip.h is what a C, Rust or cgo binding reads: it must compile as C11 on its own, and the two
    structs that cross the boundary (apk_plan, apk_attn_prologue) must have the layout the ctypes mirror assumes."""
    import shutil

    lib, _ = _lib()
    cc = shutil.which("gcc") or shutil.which("cc")
    assert cc, "no C compiler"
    inc = os.path.join(ROOT, "include")
    subprocess.check_call([cc, "-std=c11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c",
                           os.path.join(inc, "apk_hip.h")])
    fields = {"apk_plan": [f[0] for f in lib.Plan._fields_], "apk_attn_prologue": [f[0] for f in lib.AttnPrologue._fields_]}
    src = ['#include <stddef.h>', '#include <stdio.h>', '#include "apk_hip.h"', "int main(void) {"]
    for st, names in fields.items():
        src.append(f'    printf("{st} %zu\\n", sizeof({st}));')
        for f in names:
            src.append(f'    printf("{st}.{f} %zu\\n", offsetof({st}, {f}));')
    src += ["    return 0;", "}"]
    cfile, exe = tmp_path / "layout.c", tmp_path / "layout"
    cfile.write_text("\n".join(src))
    subprocess.check_call([cc, "-std=c11", f"-I{inc}", "-o", str(exe), str(cfile)])
    got = dict(line.rsplit(" ", 1) for line in subprocess.check_output([str(exe)], text=True).splitlines())
    for st, cls in (("apk_plan", lib.Plan), ("apk_attn_prologue", lib.AttnPrologue)):
        assert int(got[st]) == C.sizeof(cls), st
        for f in fields[st]:
            assert int(got[f"{st}.{f}"]) == getattr(cls, f).offset, (st, f)

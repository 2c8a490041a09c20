"""The Rust binding printed in the integration guide (GUIDE below) against include/apk_hip.h: every exported function is declared there
once, with the same number of arguments and the same type for each, and the two #[repr(C)] structs list the header's
fields in the header's order.  (Rust is not in this image, so the binding cannot be compiled here; this keeps the
text a maintainer would paste from drifting away from the header it binds.)"""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GUIDE = "INTEGRATION.md"


def _strip_c_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _c_type_to_rust(ctype):
    """'const float*' -> '*const f32' and so on, for the handful of types the header uses."""
    t = " ".join(ctype.replace("*", " * ").split())
    stars = t.count("*")
    const = t.startswith("const ")
    base = t.replace("const ", "").replace("*", "").strip()
    scalar = {
        "void": "c_void", "char": "c_char", "int": "c_int", "unsigned": "c_uint", "float": "f32",
        "size_t": "usize", "uint32_t": "u32", "uint64_t": "u64",
        "apk_ctx": "apk_ctx", "apk_graph": "apk_graph", "apk_plan": "apk_plan", "apk_attn_prologue": "apk_attn_prologue",
    }[base]
    if stars == 0:
        return scalar
    if stars == 1:
        return ("*const " if const else "*mut ") + scalar
    assert stars == 2 and not const
    return "*mut *mut " + scalar


def _split_c_arg(arg):
    """'const float* qw' -> ('const float*', 'qw')"""
    m = re.match(r"^(.*?)([A-Za-z_][A-Za-z0-9_]*)$", arg.strip(), flags=re.S)
    return m.group(1).strip(), m.group(2)


def header_functions():
    text = _strip_c_comments(open(os.path.join(ROOT, "include", "apk_hip.h")).read())
    fns = {}
    for ret, name, args in re.findall(r"([A-Za-z_][A-Za-z0-9_ \*]*?)\b(apk_[a-z0-9_]+)\s*\(([^;{)]*)\)\s*;", text, flags=re.S):
        args = args.strip()
        arg_types = [] if args in ("", "void") else [_c_type_to_rust(_split_c_arg(a)[0]) for a in args.split(",")]
        assert name not in fns, f"{name} is declared twice in the header"
        fns[name] = (_c_type_to_rust(ret.strip()), arg_types)
    return fns


def header_struct(name):
    text = _strip_c_comments(open(os.path.join(ROOT, "include", "apk_hip.h")).read())
    body = re.search(r"typedef struct " + name + r"\s*\{(.*?)\}\s*" + name + r"\s*;", text, flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        m = re.match(r"^(.*?)([A-Za-z_][A-Za-z0-9_]*(?:\s*,\s*[A-Za-z_][A-Za-z0-9_]*)*)(\[\d+\])?$", decl, flags=re.S)
        ctype, names, arr = m.group(1).strip(), m.group(2), m.group(3)
        for n in names.split(","):
            rt = _c_type_to_rust(ctype)
            fields.append((n.strip(), f"[{rt}; {arr[1:-1]}]" if arr else rt))
    return fields


def rust_binding():
    md = open(os.path.join(ROOT, GUIDE)).read()
    start = md.index("// crates/allpaka-hip-sys/src/lib.rs")
    block = md[start:md.index("```", start)]
    block = re.sub(r"//[^\n]*", "", block)
    return block


def rust_functions(block):
    ext = block[block.index('extern "C" {'):]
    fns = {}
    for name, args, ret in re.findall(r"pub fn (apk_[a-z0-9_]+)\s*\(([^)]*)\)\s*(?:->\s*([^;]+))?;", ext, flags=re.S):
        arg_types = []
        for a in [x for x in args.split(",") if x.strip()]:
            arg_types.append(" ".join(a.split(":", 1)[1].split()))
        assert name not in fns, f"{name} is bound twice"
        fns[name] = (" ".join((ret or "()").split()), arg_types)
    return fns


def rust_struct(block, name):
    body = re.search(r"pub struct " + name + r"\s*\{(.*?)\}", block, flags=re.S).group(1)
    return [(n, " ".join(t.split())) for n, t in re.findall(r"pub ([a-z_0-9]+)\s*:\s*([^,}]+?)\s*(?:,|$)", body, flags=re.S)]


def test_every_header_function_is_bound_with_the_same_arguments():
    c = header_functions()
    r = rust_functions(rust_binding())
    assert len(c) >= 60  # the parser found the header's declarations at all
    assert sorted(set(c) - set(r)) == [], "declared in include/apk_hip.h, missing from the binding"
    assert sorted(set(r) - set(c)) == [], "bound, but not in include/apk_hip.h"
    for name, (ret, args) in c.items():
        rret, rargs = r[name]
        assert len(rargs) == len(args), f"{name}: {len(args)} arguments in the header, {len(rargs)} in the binding"
        assert rargs == args, f"{name}: header {args}, binding {rargs}"
        assert rret == ret, f"{name}: returns {ret} in the header, {rret} in the binding"


def test_repr_c_structs_follow_the_header_field_for_field():
    block = rust_binding()
    for name in ("apk_attn_prologue", "apk_plan"):
        assert rust_struct(block, name) == header_struct(name), name


def test_the_arm_has_an_item_for_every_entry_of_the_stub_arm():
    """The names are the public functions of gpu/stub.rs:37-217 of the reference, frozen here as data."""
    stub_entries = """attach detach is_attached memory_architecture init_error residency_status arena_bytes stats gpu_time_stats
        set_rope_inv_freq has_device_rope_freq prefer_gpu_embed can_embed_on_gpu matvec matvec_batch ffn_batch
        ffn_batch_grouped wrap_region upload_region_range download_region_range decode_attention_capacity_safe
        minimum_kv_capacity attend attend_batch attend_project attn_block decode_token_checked decode_token
        decode_greedy_continue prefill_begin prefill_replay prefill_graph_key multi_stage prefill_end prefill_end_output
        prefill_abort prefill_attn_block prefill_gdn_block shared_activation_stats set_rope_inv_freq_swa set_quant_gemm
        set_attn_window""".split()
    md = open(os.path.join(ROOT, GUIDE)).read()
    start = md.index("// crates/allpaka-backend/src/gpu/hip/mod.rs")
    arm = md[start:md.index("\n```", start)]
    defined = set(re.findall(r"^pub fn ([a-z_0-9]+)", arm, flags=re.M)) | set(re.findall(r"pub use super::common::([a-z_]+);", arm))
    assert [e for e in stub_entries if e not in defined] == []
    assert "pub struct SharedRegion" in arm
    # every apk_ call the arm makes exists
    c = header_functions()
    used = set(re.findall(r"sys::(apk_[a-z0-9_]+)\(", arm))
    assert used and sorted(used - set(c)) == []


def test_the_printed_build_script_builds_every_source_the_makefile_links():
    """The library links what allpaka_amd/csrc/Makefile says it links; the build.rs printed for the Rust side must
    name each of those sources (or the object built from it), or the crate would fail to link."""
    mk = open(os.path.join(ROOT, "allpaka_amd", "csrc", "Makefile")).read()
    link = re.search(r"^\$\(OUT\):.*\n\t(.*)$", mk, flags=re.M).group(1)
    linked = re.findall(r"\b(apk_[a-z_]+\.(?:cpp|S|o|hip))\b", link)
    assert "apk_host.cpp" in linked and "apk_embed.S" in linked and len(linked) >= 3
    # an object stands for the source its rule compiles; the embedded code object for apk_kernels.hip
    sources = set()
    for f in linked:
        if f.endswith(".o"):
            rule = re.search(r"^" + re.escape(f) + r":\s*(\S+)", mk, flags=re.M)
            assert rule, f"no rule for {f}"
            sources.add(rule.group(1))
        else:
            sources.add(f)
    sources.add("apk_kernels.hip")
    md = open(os.path.join(ROOT, GUIDE)).read()
    start = md.index("// crates/allpaka-hip-sys/build.rs")
    build_rs = md[start:md.index("\n```", start)]
    missing = sorted(f for f in sources if f not in build_rs)
    assert missing == [], f"build.rs in {GUIDE} does not build {missing}"
    # every file it names exists in this repository
    for f in re.findall(r"\{src\}/(apk_[a-z_]+\.[a-zA-Z]+)", build_rs):
        assert os.path.exists(os.path.join(ROOT, "allpaka_amd", "csrc", f)), f


def test_every_entry_named_in_the_mapping_tables_exists():
    md = open(os.path.join(ROOT, GUIDE)).read()
    c = header_functions()
    structs = {"apk_attn_prologue", "apk_plan", "apk_ctx", "apk_graph", "apk_hip", "apk_status", "apk_dq_fmt", "apk_kernels", "apk_embed", "apk_host", "apk_noalloc", "apk_noalloc_setup"}
    named = set(re.findall(r"\bapk_[a-z0-9_]+\b", md))
    unknown = sorted(n for n in named if n not in c and n not in structs)
    assert unknown == [], unknown

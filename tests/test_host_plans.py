"""No-GPU checks of the host's launch shapes: the apk_plan_* functions return what the entries launch
(kernel, grid, workgroup size) as pure functions of the sizes, so every shape can be checked here for the
things a wrong launch would break on the device: a kernel that exists in the code object, a workgroup
within the kernel's launch bound, a grid that covers every row / tile / head exactly once and no more
than a partial workgroup beyond, and the declines of the entries for sizes they do not take."""
import ctypes as C
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32, F16 = 0, 1


@pytest.fixture(scope="module")
def L():
    import allpaka_amd.lib as lib

    if not os.path.exists(lib.lib_path()):
        subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "allpaka_amd", "csrc")])
    return lib.load()


@pytest.fixture(scope="module")
def kernels(L):
    buf = C.create_string_buffer(80)
    names = []
    for i in range(L.apk_kernel_count()):
        assert L.apk_kernel_name(i, buf, 80) == 0
        names.append(buf.value.decode())
    assert len(names) == len(set(names)) and len(names) > 100
    assert L.apk_kernel_name(len(names), buf, 80) == 4  # out of range
    return set(names)


@pytest.fixture(scope="module")
def bounds():
    """Launch bound (.max_flat_workgroup_size) of every kernel, read from the code object's metadata."""
    tool = "/opt/rocm/llvm/bin/llvm-readelf"
    co = os.path.join(ROOT, "allpaka_amd", "csrc", "apk_kernels.hsaco")
    if not (os.path.exists(tool) and os.path.exists(co)):
        pytest.skip("no llvm-readelf or no code object next to the sources")
    work = os.path.join(ROOT, "tests", "__pycache__", "co")
    os.makedirs(work, exist_ok=True)
    elf = co
    if open(co, "rb").read(4) != b"\x7fELF":  # an offload bundle: take the gfx950 member out
        bundler = "/opt/rocm/llvm/bin/clang-offload-bundler"
        if not os.path.exists(bundler):
            pytest.skip("no clang-offload-bundler")
        elf = os.path.join(work, "apk_kernels.gfx950.elf")
        subprocess.check_call([bundler, "--unbundle", "--type=o", f"--input={co}", f"--output={elf}",
                               "--targets=hipv4-amdgcn-amd-amdhsa--gfx950"])
    notes = subprocess.run([tool, "--notes", elf], capture_output=True, text=True, check=True).stdout
    out = {}
    for block in notes.split("- .agpr_count:")[1:]:
        name = re.search(r"\.name:\s+(\S+)", block)
        bound = re.search(r"\.max_flat_workgroup_size:\s+(\d+)", block)
        if name and bound:
            out[name.group(1)] = int(bound.group(1))
    shutil.rmtree(work, ignore_errors=True)
    assert len(out) > 100, "metadata not parsed"
    return out


def plan(fn, *args):
    import allpaka_amd.lib as lib

    p = lib.Plan()
    rc = fn(*args, C.byref(p))
    return rc, p


def common(p, kernels, bounds):
    name = p.kernel.decode()
    assert name in kernels, name
    assert p.block % 64 == 0 and 64 <= p.block <= bounds[name], (name, p.block, bounds[name])
    assert 1 <= p.grid < 2**31
    return name


TILE_COUNTS = [1, 2, 3, 4, 5, 6, 8, 10, 12, 16, 20]  # 16-byte tiles per lane the tiled kernels are built for
ROW_LENGTHS = [8, 16, 24, 64, 104, 128, 200, 256, 264, 512, 768, 1000, 1024, 1032, 1536, 2048, 2560, 3072, 3584, 4096, 4100, 5120,
               6144, 7168, 8192, 10240, 12288, 16384, 20480, 20488, 32768, 65536, 7, 9, 1001, 5121]
ROW_COUNTS = [1, 2, 6, 7, 8, 15, 16, 17, 33, 64, 100, 256, 511, 512, 1000, 1024, 2047, 2048, 2049, 2061, 3072, 4095, 4096, 4097,
              6000, 8191, 8192, 8193, 20000, 100000, 2**31 - 1]


@pytest.mark.parametrize("post", [False, True])
def test_add_rmsnorm_plans_cover_every_row_once(L, kernels, bounds, post):
    """post: the sandwich-norm entry (its tiled kernels hold the delta through one more reduction: at most 10 tiles
    per lane; rows outside the tiled kernels are planned as the plain entry plans them, and run as two steps)."""
    seen = set()
    fn = L.apk_plan_postnorm_add_rmsnorm_rows if post else L.apk_plan_add_rmsnorm_rows
    for dtype, es in ((F32, 4), (F16, 2)):
        vec = 16 // es
        for n in ROW_LENGTHS:
            for rows in ROW_COUNTS:
                rc, p = plan(fn, n, rows, dtype)
                assert rc == 0, (n, rows, dtype)
                name = common(p, kernels, bounds)
                seen.add(re.sub(r"_(c|l)\d+$", "", name).replace("apk_postnorm_add_rmsnorm", "apk_add_rmsnorm"))
                if post and "ragged" not in name and "small" not in name:
                    assert name.startswith("apk_postnorm_add_rmsnorm_") and p.tiles_per_lane <= 10
                nchunks = n // vec
                if "ragged" in name:  # not whole tiles, or more than the register-tiled kernels hold (20480 elements)
                    assert n % vec or n > (20480 if not post else 10240 * (2 if dtype == F16 else 1))
                    assert p.grid == rows and p.block == 256
                    continue
                assert n % vec == 0
                if "small" in name:
                    assert nchunks <= 32 and rows >= 16 and p.lanes_per_row >= nchunks and p.lanes_per_row in (4, 8, 16, 32)
                    assert p.rows_per_block == 4 * (64 // p.lanes_per_row)
                    assert (p.grid - 1) * p.rows_per_block < rows <= p.grid * p.rows_per_block
                    continue
                assert name.endswith(f"_c{p.tiles_per_lane}")
                slots = p.waves_per_row * 64 * p.tiles_per_lane
                assert slots >= nchunks > (p.waves_per_row - 1) * 64 * p.tiles_per_lane  # covered, and no idle wave
                if p.tiles_per_lane > 2:  # the smallest tile count the kernels come in that needs no more waves
                    smaller = max(c for c in TILE_COUNTS if c < p.tiles_per_lane)
                    assert nchunks > p.waves_per_row * 64 * smaller
                if p.rows_per_block > 1:
                    assert p.waves_per_row == 1 and p.block == 64 * p.rows_per_block and rows >= 8192
                    assert (p.grid - 1) * p.rows_per_block < rows <= p.grid * p.rows_per_block
                else:
                    assert p.grid == rows and p.block == 64 * p.waves_per_row
                # a batch beyond one resident round of long waves takes short ones
                if rows * p.waves_per_row > 4096 and nchunks <= 2048:
                    if post and dtype == F16:  # the sandwich norm of fp16 rows: 3, 4 or 5 tiles, whichever pads the row least
                        assert p.tiles_per_lane <= 5, (n, rows, name)
                        pads = {c: -(-nchunks // (64 * c)) * 64 * c - nchunks for c in (3, 4, 5)
                                if -(-nchunks // (64 * c)) * 64 <= (256 if c == 5 else 512)}
                        if nchunks > 128 and pads:  # (a row of at most two tiles per lane of one wave stays that)
                            assert p.tiles_per_lane >= 3 and slots - nchunks == min(pads.values()), (n, rows, name, pads)
                    else:
                        assert p.tiles_per_lane <= 2, (n, rows, dtype, name)
    assert seen == {"apk_add_rmsnorm_f32", "apk_add_rmsnorm_f16", "apk_add_rmsnorm_small_f32", "apk_add_rmsnorm_small_f16",
                    "apk_add_rmsnorm_ragged_f32", "apk_add_rmsnorm_ragged_f16"}
    # the declines of the entry, and the no-op
    assert plan(fn, 1024, 4, 7)[0] == 1
    assert plan(fn, 0, 4, F32)[0] == 2
    assert plan(fn, 1024, 2**31, F32)[0] == 2
    rc, p = plan(fn, 1024, 0, F32)
    assert rc == 0 and p.grid == 0 and p.kernel == b""
    assert fn(1024, 4, F32, None) == 3


def plan_attn(L, rows, n_q, n_kv, hd, rot, style, dtype, kv, bias, norm=True):
    """The struct form of the same plan: biases and the cache store are asked for by non-NULL pointers."""
    import allpaka_amd.lib as lib

    a = lib.AttnPrologue()
    a.rows, a.n_q, a.n_kv, a.head_dim, a.rot_dim, a.adjacent_pairs, a.dtype = rows, n_q, n_kv, hd, rot, style, dtype
    if kv:
        a.k_cache = a.v_cache = a.cache_pos = a.v = 16
        a.capacity = 1
    if bias:
        a.q_bias = a.k_bias = 16
    if norm:
        a.k_norm = 16
    p = lib.Plan()
    return L.apk_plan_attn_prologue_rows(C.byref(a), C.byref(p)), p


@pytest.mark.parametrize("bias,norm", [(False, True), (True, True), (False, False), (True, False)])
def test_qknorm_rope_plans_cover_every_head(L, kernels, bounds, bias, norm):
    """bias: the kernels that add the projection biases on the way; norm = False: no norm weight for q or k, the
    kernels without statistics."""
    for dtype, es in ((F32, 4), (F16, 2)):
        for hd, rot, style in ((64, 64, 0), (128, 128, 0), (256, 256, 0), (128, 64, 0), (96, 96, 0), (128, 128, 1), (80, 0, 0), (2, 2, 1),
                               (128, 64, 1), (256, 64, 0), (128, 8, 0), (128, 8, 1), (128, 0, 0), (64, 36, 1), (64, 48, 0)):
            for n_q, n_kv in ((64, 8), (32, 8), (16, 8), (40, 8), (28, 4), (8, 1), (1, 0), (0, 3), (12, 2), (96, 8), (5, 5)):
                for rows in (1, 6, 64, 255, 512, 2048, 2061, 8192, 100000):
                    for kv in (0, 1):
                        rc, p = plan_attn(L, rows, n_q, n_kv, hd, rot, style, dtype, kv, bias, norm)
                        if not bias and norm:  # the struct form and the flat form are one plan
                            rc2, p2 = plan(L.apk_plan_qknorm_rope, rows, n_q, n_kv, hd, rot, style, dtype, kv)
                            assert (rc2, bytes(p2)) == (rc, bytes(p))
                        epl = 16 // es  # elements of a lane's 16-byte tile
                        tiled = hd in (64, 128, 256) and rot > 0 and (rot % epl == 0 if style else (rot // 2) % epl == 0)
                        if kv and not tiled:
                            assert rc == 1
                            continue
                        if kv and n_kv == 0:
                            assert rc == 2
                            continue
                        assert rc == 0, (rows, n_q, n_kv, hd, rot, style, dtype, kv)
                        name = common(p, kernels, bounds)
                        waves_launched = p.grid * (p.block // 64)
                        if not tiled:
                            assert "generic" in name and waves_launched >= rows * (n_q + n_kv) > waves_launched - 4
                            continue
                        assert name == (f"apk_{'qknorm_rope' if norm else 'rope'}_{'pairs_' if style else ''}{'kv_' if kv else ''}{'bias_' if bias else ''}"
                                        f"{'f32' if dtype == F32 else 'f16'}_hd{hd}_i{p.tiles_per_lane}")
                        lph = hd // 2 // (16 // es)  # lanes per head
                        hpw = 64 // lph
                        # one pass per wave; fp16 kernels run as two-wave workgroups (their constants sit in LDS)
                        assert p.lanes_per_row == lph and p.tiles_per_lane == 1 and p.block == (128 if dtype == F16 else 256)
                        q_waves = -(-n_q // hpw)
                        k_waves = -(-n_kv // hpw)
                        # with the cache store the v rows are narrowed by waves of their own
                        assert p.waves_per_row == q_waves + k_waves * (2 if kv else 1) and p.items == rows * p.waves_per_row
                        assert waves_launched >= p.items > waves_launched - 4
    assert plan(L.apk_plan_qknorm_rope, 4, 8, 2, 128, 126, 0, 9, 0)[0] == 1  # dtype
    assert plan(L.apk_plan_qknorm_rope, 4, 8, 2, 128, 127, 0, F32, 0)[0] == 2  # odd rotary width
    assert plan(L.apk_plan_qknorm_rope, 4, 8, 2, 128, 130, 0, F32, 0)[0] == 2  # wider than the head
    assert plan(L.apk_plan_qknorm_rope, 4, 8, 2, 0, 0, 0, F32, 0)[0] == 2
    assert plan(L.apk_plan_qknorm_rope, 4, 70000, 2, 128, 128, 0, F32, 0)[0] == 2
    rc, p = plan(L.apk_plan_qknorm_rope, 0, 8, 2, 128, 128, 0, F32, 0)
    assert rc == 0 and p.grid == 0
    assert L.apk_plan_attn_prologue_rows(None, C.byref(p)) == 3


def test_scatter_plans_group_the_hits_of_a_slice_on_one_xcd(L, kernels, bounds):
    for dtype, es in ((F32, 4), (F16, 2)):
        for cols in (16 // es, 64, 520, 2048, 3600, 4096, 8200, 65536):
            if cols * es % 16:
                continue
            for rows in (1, 3, 9, 600, 1024, 4099, 100000):
                for k in (1, 2, 8, 64):
                    rc, p = plan(L.apk_plan_scatter_rows, rows, k, cols, dtype)
                    if rc != 0:
                        assert rc == 2 and rows * k * -(-cols * es // 16 // 256) >= 2**31 // 2, (rows, k, cols)
                        continue
                    name = common(p, kernels, bounds)
                    row_vecs = cols * es // 16
                    assert name == f"apk_scatter_rows_t{p.tiles_per_lane}" and p.block == 256
                    assert (p.tiles_per_lane == 1) == (rows * k * cols * es >= 64 << 20)
                    per_slice = 256 * p.tiles_per_lane
                    assert p.slices_per_row * per_slice >= row_vecs > (p.slices_per_row - 1) * per_slice
                    assert p.items == rows * p.slices_per_row
                    # workgroup b takes item (b % 8) + 8 * ((b // 8) // k), hit (b // 8) % k: every (item, hit) once
                    assert p.grid == -(-p.items // 8) * 8 * k
                    if p.items * k <= 4096:
                        got = sorted(((b % 8) + 8 * ((b // 8) // k), (b // 8) % k) for b in range(p.grid))
                        got = [g for g in got if g[0] < p.items]
                        assert got == [(i, j) for i in range(p.items) for j in range(k)]
    assert plan(L.apk_plan_scatter_rows, 4, 2, 3, F32)[0] == 2  # a row that is not whole 16-byte tiles
    assert plan(L.apk_plan_scatter_rows, 4, 2, 64, 5)[0] == 1
    rc, p = plan(L.apk_plan_scatter_rows, 0, 2, 64, F32)
    assert rc == 0 and p.grid == 0


def test_embed_plans_cover_every_tile_of_a_row(L, kernels, bounds):
    names = ["q4k", "q5k", "q6k", "q8_0", "q2k", "q3k", "q5_0", "f16", "f32", "bf16"]
    block_elems = [256, 256, 256, 32, 256, 256, 32, 1, 1, 1]
    for fmt in range(10):
        for out_dtype, oes in ((F32, 4), (F16, 2)):
            for n_in in (256, 512, 1024, 2048, 4096, 5120, 8192, 12288, 16384, 20480, 32768, 64, 96, 4104, 8):
                for t in (1, 6, 512, 2048, 100000):
                    rc, p = plan(L.apk_plan_embed_rows, fmt, n_in, t, out_dtype)
                    if n_in % block_elems[fmt] or n_in % 8 or not L.apk_can_embed(fmt, n_in):
                        assert rc == 1, (fmt, n_in)
                        continue
                    assert rc == 0, (fmt, n_in, t)
                    name = common(p, kernels, bounds)
                    assert name == f"apk_embed_{names[fmt]}_{'f32' if out_dtype == F32 else 'f16'}"
                    assert p.block <= 256
                    if fmt in (1, 2, 4, 5):  # 8 lanes per super-block, super-blocks numbered across the batch: no idle lane but at the end
                        lanes = t * (n_in // 256) * 8
                        assert p.items * 8 == lanes and p.slices_per_row == 0
                        assert p.block == min(256, -(-lanes // 64) * 64)
                        assert p.grid * p.block >= lanes > (p.grid - 1) * p.block
                        assert p.tiles_per_lane * 8 * (16 // oes) == 256
                        continue
                    assert p.grid == t * p.slices_per_row
                    tiles = n_in // (16 // oes)
                    if fmt == 0:  # Q4_K: the workgroup loops over the row's super-blocks, 8 lanes each
                        assert p.slices_per_row == 1 and p.block == min(256, -(-(n_in // 256 * 8) // 64) * 64)
                    elif fmt in (3, 6, 8):  # four output tiles per lane
                        assert p.tiles_per_lane == 4
                        assert p.slices_per_row * p.block * 4 >= tiles > (p.slices_per_row - 1) * p.block * 4
                    else:  # F16 / BF16: the row staged in LDS
                        assert p.slices_per_row == 1 and p.shmem == 2 * n_in + 32 <= 64 * 1024
    assert plan(L.apk_plan_embed_rows, 7, 32768, 4, F32)[0] == 1  # an F16 row beyond the staging buffer
    assert plan(L.apk_plan_embed_rows, 11, 256, 4, F32)[0] == 1
    assert plan(L.apk_plan_embed_rows, 0, 256, 4, 3)[0] == 1
    rc, p = plan(L.apk_plan_embed_rows, 0, 256, 0, F32)
    assert rc == 0 and p.grid == 0

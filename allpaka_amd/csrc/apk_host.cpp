// Host side of libapk_hip.so: the C ABI declared in include/apk_hip.h.
//
// A thin runtime: one embedded gfx950 code object loaded with hipModuleLoadData,
// one hipStream, argument validation that DECLINES (positive status) instead of
// failing, and hipModuleLaunchKernel.  No device code in this translation unit:
// it builds with a plain host C++ compiler against the HIP runtime API.
#include "apk_hip.h"
#include "apk_internal.h"

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstring>
#include <map>
#include <set>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

extern "C" const unsigned char apk_kernels_co[];
extern "C" const unsigned char apk_kernels_co_end[];

namespace {

thread_local char g_err[512] = "";

int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return status;
}
int hip_fail(hipError_t e, const char* what) {
    return fail(-(int)e, "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
}
#define HIP_TRY(expr)                                  \
    do {                                               \
        hipError_t e_ = (expr);                        \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

uint64_t now_ns() {
    return (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(
               std::chrono::steady_clock::now().time_since_epoch())
        .count();
}

struct Mapping {
    void* dev;
    size_t len;
    size_t owners;  // attaches of exactly this (base, len) not yet detached
    uint64_t serial;  // the context's clock when the copy was made (graphs recorded later may hold addresses inside it)
};

// Every kernel of the embedded code object, resolved once at apk_init so that a
// missing symbol fails there and not at the first launch.
const int kAddnormTiles[] = {1, 2, 3, 4, 5, 6, 8, 10, 12, 16, 20};  // 16-byte tiles per lane
const int kAddnormBound[] = {1024, 1024, 512, 512, 256, 256, 256, 256, 256, 256, 256};  // launch bound of each
const int kQkIters[] = {1};
const int kQkHeadDims[] = {64, 128, 256};

std::vector<std::string> all_kernel_names() {
    std::vector<std::string> v = {"apk_swiglu_f32", "apk_swiglu_f16", "apk_geglu_tanh_f32", "apk_geglu_tanh_f16", "apk_rope_table", "apk_embed_q4k_f32",
                                  "apk_embed_q4k_f16", "apk_embed_q8_0_f32", "apk_embed_q8_0_f16", "apk_route_topk",
                                  "apk_moe_permute", "apk_gather_rows", "apk_scatter_rows_t1", "apk_scatter_rows_t2", "apk_argmax_rows", "apk_add_rmsnorm_ragged_f32", "apk_add_rmsnorm_ragged_f16", "apk_copy",
                                  "apk_qknorm_rope_generic_f32", "apk_qknorm_rope_generic_f16", "apk_qknorm_rope_pos_f32", "apk_qknorm_rope_pos_f16", "apk_route_topk_wide", "apk_route_topk_e64", "apk_route_topk_e128", "apk_route_group_small_e64", "apk_route_group_small_e128",
                                  "apk_route_group_small_e256", "apk_route_group_small_e1024", "apk_add_assign_f32", "apk_add_assign_f16", "apk_add_scaled_f32", "apk_add_scaled_f16", "apk_softmax_rows", "apk_moe_count", "apk_moe_rank",
                                  "apk_add_bias_rows_f32", "apk_add_bias_rows_f16", "apk_moe_shared_hits", "apk_cast_f32_f16", "apk_cast_f16_f32", "apk_zero_u64"};
    for (const char* t : {"f32", "f16"}) {
        for (const char* f : {"q5k", "q6k", "q2k", "q3k", "q5_0", "f16", "f32", "bf16"}) v.push_back(std::string("apk_embed_") + f + "_" + t);
        for (int c : kAddnormTiles) v.push_back(std::string("apk_add_rmsnorm_") + t + "_c" + std::to_string(c));
        for (int c : kAddnormTiles) v.push_back(std::string("apk_postnorm_add_rmsnorm_") + t + "_c" + std::to_string(c));
        for (int l : {4, 8, 16, 32}) v.push_back(std::string("apk_add_rmsnorm_small_") + t + "_l" + std::to_string(l));
        for (int c : {1, 2, 4}) v.push_back(std::string("apk_combine_add_rmsnorm_") + t + "_c" + std::to_string(c));
        for (int hd : kQkHeadDims) v.push_back(std::string("apk_layer_prologue_") + t + "_hd" + std::to_string(hd));
        for (const char* pfx : {"apk_qknorm_rope_", "apk_rope_"})  // with a norm weight for q and / or k; with none
            for (int hd : kQkHeadDims)
                for (int it : kQkIters)
                    for (const char* style : {"", "pairs_"})
                        for (const char* kv : {"", "kv_"})
                            for (const char* bias : {"", "bias_"})
                                v.push_back(std::string(pfx) + style + kv + bias + t + "_hd" + std::to_string(hd) + "_i" + std::to_string(it));
    }
    return v;
}

}  // namespace

struct apk_ctx {
    int device = 0;
    hipModule_t module = nullptr;
    hipStream_t stream = nullptr;
    std::unordered_map<std::string, hipFunction_t> fn;
    std::unordered_map<uint32_t, hipFunction_t> fn_by_key;  // (op, variant) -> function: no name building on the hot path
    uint32_t* fault_dev = nullptr;  // device status word
    uint32_t* ids_stage_host = nullptr;  // pinned staging for host-side token ids
    uint32_t* ids_stage_dev = nullptr;
    size_t ids_stage_cap = 0;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    void* argmax_scratch = nullptr;  // one 128-byte line per row: u64 running best + u32 arrivals; zero between calls
    size_t argmax_rows_cap = 0;
    bool capturing = false;        // between apk_capture_begin and apk_capture_end / _abort
    size_t capture_nodes = 0;      // launches recorded so far
    bool capture_argmax = false;   // the recording holds the argmax scratch address
    size_t graphs_with_argmax = 0; // live graphs that do: the scratch must not move under them
    uint32_t* permute_counts = nullptr;  // counts[part][expert] of the two-launch grouping
    size_t permute_counts_cap = 0;       // in u32
    bool capture_permute = false;
    size_t graphs_with_permute = 0;
    std::set<apk_graph*> live_graphs;  // recorded graphs not yet destroyed: they hold device addresses, also inside attached mappings
    uint64_t clock = 0;  // counts attaches that copied and recordings that ended: orders a graph against a mapping
    std::mutex mu;
    std::map<uintptr_t, Mapping> attached;
    std::atomic<uint64_t> calls{0}, dispatches{0}, encode_ns{0}, wait_ns{0};
};

int apk_fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return status;
}
int apk_ctx_device(apk_ctx* c) { return c ? c->device : -1; }

struct apk_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    size_t nodes = 0;
    bool uses_argmax = false;
    bool uses_permute = false;
    uint64_t born = 0;   // the context's clock when the recording ended
    bool stale = false;  // a mapping that was attached while this was recorded has been freed since: never replayed again
};

namespace {

struct CallScope {  // counts one ABI call and its host-side encode time
    apk_ctx* c;
    uint64_t t0;
    std::lock_guard<std::mutex> lock;
    explicit CallScope(apk_ctx* ctx) : c(ctx), t0(now_ns()), lock(ctx->mu) { c->calls++; }
    ~CallScope() { c->encode_ns += now_ns() - t0; }
};

int launch_fn(apk_ctx* c, hipFunction_t f, const char* what, unsigned grid, unsigned block, unsigned shmem, void** args) {
    hipError_t e = hipModuleLaunchKernel(f, grid, 1, 1, block, 1, 1, shmem, c->stream, args, nullptr);
    if (e != hipSuccess) return hip_fail(e, what);
    if (c->capturing) c->capture_nodes++;  // recorded, not run: counted when the graph is replayed
    else c->dispatches++;
    return APK_OK;
}

int launch(apk_ctx* c, const std::string& k, unsigned grid, unsigned block, unsigned shmem, void** args) {
    if (grid == 0) return APK_OK;
    auto it = c->fn.find(k);
    if (it == c->fn.end()) return fail(APK_DECLINE_UNSUPPORTED, "no kernel %s in the code object", k.c_str());
    return launch_fn(c, it->second, k.c_str(), grid, block, shmem, args);
}

// The same for the ops of the decode chain, where the host's cost per launch is what bounds
// the chain: the kernel of an (op, variant) pair is looked up by an integer; its name is built
// only the first time.
enum OpId : uint32_t { OP_GEGLU = 20, OP_SWIGLU = 1, OP_ADDNORM, OP_QKROPE, OP_QKROPE_KV, OP_PROLOGUE, OP_ADD_ASSIGN, OP_EMBED, OP_ARGMAX };
template <typename NameFn>
int launch_keyed(apk_ctx* c, OpId op, uint32_t variant, NameFn&& name, unsigned grid, unsigned block, unsigned shmem,
                 void** args) {
    if (grid == 0) return APK_OK;
    const uint32_t key = ((uint32_t)op << 24) | (variant & 0xffffffu);
    auto it = c->fn_by_key.find(key);
    if (it == c->fn_by_key.end()) {
        const std::string k = name();
        auto byname = c->fn.find(k);
        if (byname == c->fn.end()) return fail(APK_DECLINE_UNSUPPORTED, "no kernel %s in the code object", k.c_str());
        it = c->fn_by_key.emplace(key, byname->second).first;
    }
    return launch_fn(c, it->second, "hipModuleLaunchKernel", grid, block, shmem, args);
}

// Entries that allocate, copy to or from the host, or wait cannot run inside a recording.
#define NOT_WHILE_CAPTURING(c, name)                                                              \
    do {                                                                                          \
        if ((c)->capturing) return fail(APK_DECLINE_CAPTURE, name ": not possible while recording"); \
    } while (0)

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }
int elem_size(int dtype) { return dtype == APK_F32 ? 4 : (dtype == APK_F16 ? 2 : 0); }

// block geometry: crates/allpaka-dtype/src/lib.rs:79-108
void block_geom(int fmt, size_t* be, size_t* bb) {
    static const size_t kBe[10] = {256, 256, 256, 32, 256, 256, 32, 1, 1, 1};
    static const size_t kBb[10] = {144, 176, 210, 34, 84, 110, 22, 2, 4, 2};
    if (fmt < 0 || fmt > 9) { *be = *bb = 0; return; }
    *be = kBe[fmt];
    *bb = kBb[fmt];
}

int set_device(apk_ctx* c) {
    HIP_TRY(hipSetDevice(c->device));
    return APK_OK;
}

// Workgroup size of the pure streaming kernels (one 16-byte tile per lane, no cross-lane work): from about a
// million tiles on, single-wave workgroups spread most evenly over the CUs and measure 1-2 % faster (SwiGLU over
// [2048 x 25600]: 49.1 -> 48.4 us in fp16, 94.5 -> 92.8 us in f32); below that four waves to a workgroup are
// ahead by as much (fewer workgroups to dispatch while the launch is short).
unsigned stream_block(uint64_t tiles) { return tiles >= (1u << 20) ? 64 : 256; }

// ---- launch plans: which kernel, how many workgroups of how many lanes, for a shape.  Pure functions of
// the sizes (no context, no GPU): the entries below launch exactly what these return, and the exported
// apk_plan_* let a host check them anywhere.
void plan_reset(apk_plan* p) { memset(p, 0, sizeof *p); }
void plan_name(apk_plan* p, const std::string& k) { snprintf(p->kernel, sizeof p->kernel, "%s", k.c_str()); }

enum { QK_TILED = 0, QK_GENERIC = 1 };
// style: 0 = NeoX pairs (i, i + rot_dim/2), 1 = adjacent pairs (2i, 2i+1); with_kv: the K/V cache store fused in
// with_bias: the kernels that also add the projection biases; with_norm = false: no norm weight for q or for k
// (the kernels without statistics)
int plan_qknorm_rope(size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, int style, int dtype, bool with_kv,
                     apk_plan* p, bool with_bias = false, bool with_norm = true) {
    plan_reset(p);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_qknorm_rope: dtype %d", dtype);
    if (head_dim == 0 || head_dim > 65536 || rot_dim % 2 || rot_dim > head_dim)
        return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope: head_dim %zu, rot_dim %zu", head_dim, rot_dim);
    // the tiled kernels: heads of 64 / 128 / 256 whose rotary width is a whole number of the lanes' 16-byte tiles
    // (adjacent pairs: a tile rotates or it does not; NeoX: the partner halves are whole tiles); no rotation at
    // all and every other geometry take the element-wise kernel
    const size_t epl_t = 16 / es;
    const bool tiled = (head_dim == 64 || head_dim == 128 || head_dim == 256) && rot_dim > 0 &&
                       (style ? rot_dim % epl_t == 0 : (rot_dim / 2) % epl_t == 0);
    if (with_kv && !tiled)
        return fail(APK_DECLINE_UNSUPPORTED, "apk_qknorm_rope_kv_store: heads of 64/128/256 with a rotary width of whole tiles only (head_dim %zu, rot_dim %zu)",
                    head_dim, rot_dim);
    if (rows == 0 || n_q + n_kv == 0) return APK_OK;
    if (with_kv && n_kv == 0) return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope_kv_store: no k heads");
    if (rows > 0x7fffffffu || n_q > 65535 || n_kv > 65535) return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope: too large");
    const char* t = dtype == APK_F32 ? "f32" : "f16";
    if (!tiled) {
        // a wave per head, element-wise: any head_dim, partial rotary, either pairing
        const uint64_t grid = ((uint64_t)rows * (n_q + n_kv) + 3) / 4;
        if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope: too large");
        p->variant = QK_GENERIC;
        plan_name(p, std::string("apk_qknorm_rope_generic_") + t);
        p->grid = (unsigned)grid;
        p->block = 256;
        p->lanes_per_row = 64;
        p->rows_per_block = 4;
        return APK_OK;
    }
    // A wave owns (row, q or k, group of HPW heads), HPW = heads per wave pass: one pass per wave.  Measured over
    // 1024..8192 rows: longer waves (two or four passes) hold more registers per resident byte and lose 2-8 % once
    // the arithmetic of a pass shows next to the stream; short waves also fill in evenly when a batch is not a whole
    // number of resident rounds.  fp16 kernels keep their constants in LDS and run as workgroups of two waves
    // (8 resident waves per SIMD); f32 kernels keep them in registers, four waves to a workgroup.
    const size_t epl = 16 / es, lph = head_dim / 2 / epl, hpw = 64 / lph;
    const size_t gk = (n_kv + hpw - 1) / hpw;
    const unsigned iter = 1;
    // with the cache store, the v rows are narrowed by waves of their own (as many as the k waves)
    const size_t waves_per_row = (n_q + hpw * iter - 1) / (hpw * iter) + gk + (with_kv ? gk : 0);
    const uint64_t waves = (uint64_t)rows * waves_per_row;
    const unsigned block = dtype == APK_F16 ? 128 : 256;
    const uint64_t grid = (waves * 64 + block - 1) / block;
    if (grid > 0x7fffffffu || waves > 0xffffffffu) return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope: too large");  // the kernels index waves in 32 bits
    p->variant = QK_TILED;
    plan_name(p, std::string(with_norm ? "apk_qknorm_rope_" : "apk_rope_") + (style ? "pairs_" : "") + (with_kv ? "kv_" : "") + (with_bias ? "bias_" : "") + t + "_hd" +
                     std::to_string(head_dim) + "_i" + std::to_string(iter));
    p->grid = (unsigned)grid;
    p->block = block;
    p->tiles_per_lane = iter;
    p->lanes_per_row = (unsigned)lph;
    p->waves_per_row = (unsigned)waves_per_row;
    p->items = (unsigned)(waves > 0xffffffffu ? 0xffffffffu : waves);
    return APK_OK;
}

enum { EMBED_Q4K = 0, EMBED_SUPERBLOCK = 1, EMBED_DIRECT = 2, EMBED_STAGED = 3 };
int plan_embed(int fmt, size_t n_in, size_t t, int out_dtype, apk_plan* p) {
    plan_reset(p);
    if (!apk_can_embed(fmt, n_in)) return fail(APK_DECLINE_UNSUPPORTED, "apk_embed_rows: fmt %d / n_in %zu", fmt, n_in);
    const int oes = elem_size(out_dtype);
    if (!oes) return fail(APK_DECLINE_UNSUPPORTED, "apk_embed_rows: out_dtype %d", out_dtype);
    if (t == 0) return APK_OK;
    if (n_in > 0x7fffffffu || t > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_embed_rows: sizes out of range");
    static const char* const kFmtName[10] = {"q4k", "q5k", "q6k", "q8_0", "q2k", "q3k", "q5_0", "f16", "f32", "bf16"};
    plan_name(p, std::string("apk_embed_") + kFmtName[fmt] + (out_dtype == APK_F32 ? "_f32" : "_f16"));
    uint64_t grid = t;
    size_t threads = 0;
    if (fmt == APK_FMT_Q4K) {
        // one workgroup per row, 8 lanes per 256-element super-block
        p->variant = EMBED_Q4K;
        threads = (n_in / 256 * 8 + 63) / 64 * 64;
        p->slices_per_row = 1;
    } else if (fmt == APK_FMT_Q6K || fmt == APK_FMT_Q5K || fmt == APK_FMT_Q2K || fmt == APK_FMT_Q3K) {
        // decoded straight from global memory, 8 lanes per 256-element super-block (the Q4_K lane layout), the
        // super-blocks numbered across the batch: workgroups of 256 lanes, none idle but in the last one
        p->variant = EMBED_SUPERBLOCK;
        const uint64_t sbs = (uint64_t)t * (n_in / 256);
        if (sbs > 0xffffffffu) return fail(APK_DECLINE_SHAPE, "apk_embed_rows: too large");
        threads = (size_t)std::min<uint64_t>(256, (sbs * 8 + 63) / 64 * 64);
        grid = (sbs * 8 + threads - 1) / threads;
        p->slices_per_row = 0;  // a workgroup is not tied to a row
        p->items = (unsigned)sbs;
        p->tiles_per_lane = (unsigned)(256 / (16 / oes) / 8);
    } else if (fmt == APK_FMT_Q8_0 || fmt == APK_FMT_Q5_0 || fmt == APK_FMT_F32) {
        // decoded straight from global memory: a lane owns 4 of the row's 16-byte output tiles; a row takes
        // one workgroup of up to 256 lanes, or several chunks of 1024 tiles
        p->variant = EMBED_DIRECT;
        const size_t tiles_per_row = n_in / (16 / oes);
        threads = ((tiles_per_row + 3) / 4 + 63) / 64 * 64;
        if (threads > 256) threads = 256;
        p->slices_per_row = (unsigned)((tiles_per_row + threads * 4 - 1) / (threads * 4));
        p->tiles_per_lane = 4;
    } else {
        // F16 / BF16: one workgroup per row, the row staged in LDS, one output tile per lane and pass
        p->variant = EMBED_STAGED;
        threads = (n_in / (16 / oes) + 63) / 64 * 64;
        p->shmem = (unsigned)(apk_row_bytes(fmt, n_in) + 32);
        p->slices_per_row = 1;
    }
    if (threads > 256) threads = 256;
    if (p->variant != EMBED_SUPERBLOCK) grid *= p->slices_per_row;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_embed_rows: too large");
    p->grid = (unsigned)grid;
    p->block = (unsigned)threads;
    return APK_OK;
}

enum { ADDNORM_RAGGED = 0, ADDNORM_SMALL = 1, ADDNORM_TILED = 2 };
int plan_add_rmsnorm(size_t n, size_t rows, int dtype, apk_plan* p, bool post = false) {
    plan_reset(p);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_add_rmsnorm_rows: dtype %d", dtype);
    if (rows == 0) return APK_OK;
    const size_t vec = 16 / es;
    if (rows > 0x7fffffffu || n > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_add_rmsnorm_rows: too large");
    if (n == 0) return fail(APK_DECLINE_SHAPE, "apk_add_rmsnorm_rows: n is 0");
    // Tiles per lane (NCH) and waves per row (W = ceil(nchunks / (64*NCH))), by batch size:
    //  * few rows (rows * W <= 2048 waves, 8 per CU): the smallest NCH, i.e. the most waves per row;
    //  * a batch that is resident all at once with a wave per row (or the fewest waves the register
    //    budget allows): that shape -- every load of the launch is in flight at once, no barrier;
    //  * a larger batch runs in several rounds of waves, and long waves then leave a long tail:
    //    two tiles per lane and W waves per row, which stays within a few per cent of a plain copy
    //    of the same bytes (6000 rows of 4096 fp16: 32.5 us against 36.7 us with a wave per row).
    // Resident waves: 16 per CU up to 10 tiles per lane (<= 128 VGPRs), 12 at 12 tiles (144 VGPRs),
    // 8 at 16 and 20 tiles (187 / 233 VGPRs).
    const size_t nchunks = n / vec;
    // (the sandwich-norm kernels hold the delta tiles through one more reduction: up to 10 tiles per lane,
    // 140 / 176 VGPRs there, so fewer resident waves)
    const int max_nch = (dtype == APK_F16 || post) ? 10 : 20;
    int nch = 0;
    size_t waves = 0;
    if (n % vec == 0) {
        for (size_t i = 0; i < sizeof kAddnormTiles / sizeof kAddnormTiles[0]; i++) {
            const int cand = kAddnormTiles[i];
            if (cand > max_nch) break;
            const size_t w = (nchunks + 64 * (size_t)cand - 1) / (64 * (size_t)cand);
            if (w * 64 > (size_t)kAddnormBound[i]) continue;
            if (nch && w >= waves) continue;  // more tiles per lane only where that saves waves (no idle tiles)
            nch = cand;
            waves = w;
            if (rows * w <= 2048) break;
        }
        const size_t resident = post ? (nch >= 10 ? (dtype == APK_F16 ? 3072 : 2048) : nch >= 8 ? 3072 : 4096)
                                     : nch >= 16 ? 2048 : nch >= 12 ? 3072 : 4096;
        if (nch > 2 && rows * waves > resident) {
            const size_t w2 = (nchunks + 127) / 128;
            if (w2 * 64 <= 1024) {
                nch = 2;
                waves = w2;
            }
            if (post && dtype == APK_F16) {
                // The sandwich norm of fp16 rows does about twice the arithmetic per tile, and its two-tile kernel
                // keeps too few bytes in flight next to it (94 registers: 5 waves of 2 x 2 KiB per SIMD): 3, 4 or 5
                // tiles per lane, whichever pads the row least (ties: the fewer waves), measured 5-44 % faster than
                // two over 1536..10240 columns and 4096..16384 rows (4096 columns: 1 % slower).  f32 rows stay at two:
                // three tiles were 2-7 % faster up to 4096 rows and up to 4 % slower beyond.
                size_t best_pad = ~(size_t)0;
                for (int cand = 5; cand >= 3; cand--) {
                    const size_t w = (nchunks + 64 * (size_t)cand - 1) / (64 * (size_t)cand);
                    if (w * 64 > (size_t)(cand == 5 ? 256 : 512)) continue;
                    const size_t pad = w * 64 * cand - nchunks;
                    if (pad < best_pad) {
                        best_pad = pad;
                        nch = cand;
                        waves = w;
                    }
                }
            }
        }
    }
    const char* t = dtype == APK_F32 ? "f32" : "f16";
    if (!nch) {
        // rows that are not whole 16-byte tiles, or longer than the tiled kernels hold in registers
        // (20 480 elements): the element-wise two-pass kernel, a workgroup per row
        p->variant = ADDNORM_RAGGED;
        plan_name(p, std::string("apk_add_rmsnorm_ragged_") + t);
        p->grid = (unsigned)rows;
        p->block = 256;
        p->waves_per_row = 4;
        return APK_OK;
    }
    if (nchunks <= 32 && rows >= 16) {
        // short rows in bulk (one head each, say): several rows per wave
        const unsigned lpr = nchunks <= 4 ? 4 : nchunks <= 8 ? 8 : nchunks <= 16 ? 16 : 32;
        const uint64_t rows_per_block = 4 * (64 / lpr);
        const uint64_t grid = (rows + rows_per_block - 1) / rows_per_block;
        if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_add_rmsnorm_rows: too large");
        p->variant = ADDNORM_SMALL;
        plan_name(p, std::string("apk_add_rmsnorm_small_") + t + "_l" + std::to_string(lpr));
        p->grid = (unsigned)grid;
        p->block = 256;
        p->lanes_per_row = lpr;
        p->rows_per_block = (unsigned)rows_per_block;
        p->tiles_per_lane = 1;
        return APK_OK;
    }
    // a wave per row: single-wave workgroups spread most evenly over the CUs (2441 rows of 4096 fp16: 14.4 us,
    // against 17.0 us as 611 workgroups of four waves); from about 8192 rows on the spread no longer matters
    // and four rows (waves) to a workgroup measure 1-3 % faster
    const unsigned rpb = (waves == 1 && rows >= 8192) ? 4 : 1;
    p->variant = ADDNORM_TILED;
    plan_name(p, std::string(post ? "apk_postnorm_add_rmsnorm_" : "apk_add_rmsnorm_") + t + "_c" + std::to_string(nch));
    p->grid = (unsigned)(rpb > 1 ? (rows + rpb - 1) / rpb : rows);
    p->block = (unsigned)(rpb > 1 ? 256 : waves * 64);
    p->tiles_per_lane = (unsigned)nch;
    p->waves_per_row = (unsigned)waves;
    p->rows_per_block = rpb;
    p->lanes_per_row = (unsigned)waves * 64;
    return APK_OK;
}

int plan_scatter(size_t rows, size_t k, size_t cols, int dtype, apk_plan* p) {
    plan_reset(p);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_scatter_rows: dtype %d", dtype);
    if (rows == 0 || k == 0 || cols == 0) return APK_OK;
    if ((cols * es) % 16) return fail(APK_DECLINE_SHAPE, "apk_scatter_rows: rows must be whole 16-byte tiles");
    if (rows > 0x7fffffffu || k > 0x7fffffffu || cols * es / 16 > 0x7fffffffu)
        return fail(APK_DECLINE_SHAPE, "apk_scatter_rows: too large");
    // one workgroup per (token, slice, hit); one 16-byte tile per lane from 64 MB of output on, two below
    // (fewer, slightly longer waves are ahead while the launch is short)
    const uint64_t row_vecs = cols * es / 16;
    const unsigned tpt = (uint64_t)rows * k * cols * es >= (64u << 20) ? 1 : 2;
    const uint64_t slices = (row_vecs + 256 * tpt - 1) / (256 * tpt);
    const uint64_t items = (uint64_t)rows * slices;
    const uint64_t grid = (items + 7) / 8 * 8 * k;
    if (items > 0xffffffffu || grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_scatter_rows: too large");
    plan_name(p, tpt == 1 ? "apk_scatter_rows_t1" : "apk_scatter_rows_t2");
    p->grid = (unsigned)grid;
    p->block = 256;
    p->tiles_per_lane = tpt;
    p->slices_per_row = (unsigned)slices;
    p->items = (unsigned)items;
    return APK_OK;
}

// the caller holds the context (CallScope).  scratch: one 128-byte line per row, zero on entry (the kernel re-arms
// it) unless clear_first asks for a fill kernel ahead of the launch.
int argmax_locked(apk_ctx* c, const float* logits, size_t rows, size_t n, uint32_t* out, void* scratch, bool clear_first) {
    if (rows == 0) return APK_OK;
    if (!logits || !out || !scratch) return fail(APK_DECLINE_NULL, "apk_argmax_rows: NULL tensor");
    if (n == 0 || n > 0xffffffffu || rows > (1u << 20)) return fail(APK_DECLINE_SHAPE, "apk_argmax_rows: sizes out of range");
    if (int rc = set_device(c)) return rc;
    if (clear_first) {
        uint64_t words = (uint64_t)rows * 16;
        void* zargs[] = {&scratch, &words};
        if (int rc = launch(c, "apk_zero_u64", (unsigned)((words + 255) / 256), 256, 0, zargs)) return rc;
    }
    // Enough workgroups per row to spread a vocabulary-sized row over the chip, and no more: the parts of a row merge
    // through two atomics on one cache line, which serialise (38 parts of 4 K logits per row: 9.4 us for 64 x 151 936
    // logits; 19 parts of 8 K logits, workgroups of 512 lanes: 9.2; 128 parts: 16).  A few rows keep the finer split.
    const unsigned block = rows >= 16 ? 512 : 256;
    size_t parts = (n + 16 * block - 1) / (16 * block);  // one pass of four 16-byte loads per lane
    if (parts > 64) parts = 64;
    if (parts < 1) parts = 1;
    while (parts > 1 && rows * parts > 8192) parts /= 2;
    uint64_t n64 = n;
    int parts_i = (int)parts;
    void* args[] = {&logits, &n64, &parts_i, &scratch, &out};
    return launch_keyed(c, OP_ARGMAX, 0, [] { return std::string("apk_argmax_rows"); }, (unsigned)(rows * parts), block, 0, args);
}

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

const char* apk_last_error(void) { return g_err; }

size_t apk_row_bytes(int fmt, size_t n_in) {
    size_t be, bb;
    block_geom(fmt, &be, &bb);
    if (!be || n_in % be) return 0;
    return n_in / be * bb;
}

int apk_can_embed(int fmt, size_t n_in) {
    // every format of the unified codes; rows must be whole 16-byte output tiles; F16 / BF16 rows
    // (the two formats still staged through LDS) must fit the 64 KiB staging buffer
    const size_t rb = apk_row_bytes(fmt, n_in);
    if (rb == 0 || n_in == 0 || n_in % 8) return 0;
    return (fmt == APK_FMT_F16 || fmt == APK_FMT_BF16) ? rb + 32 <= 64 * 1024 : 1;
}

int apk_init(int device, apk_ctx** out) {
    if (!out) return fail(APK_DECLINE_NULL, "apk_init: out is NULL");
    *out = nullptr;
    const char* no_gpu = getenv("ALLPAKA_NO_GPU");
    if (no_gpu && *no_gpu && strcmp(no_gpu, "0") != 0)
        return fail(APK_DECLINE_NO_DEVICE, "apk_init: disabled by ALLPAKA_NO_GPU");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0 || device < 0 || device >= n)
        return fail(APK_DECLINE_NO_DEVICE, "apk_init: no usable HIP device %d (count %d, %s)", device, n,
                    hipGetErrorString(e));
    apk_ctx* c = new apk_ctx();
    c->device = device;
    int rc = [&]() -> int {
        HIP_TRY(hipSetDevice(device));
        if (int rs = apk_noalloc_setup(device)) return rs;  // the address of the static scratch of apk_argmax_rows_noalloc on this device
        HIP_TRY(hipModuleLoadData(&c->module, apk_kernels_co));
        for (const std::string& name : all_kernel_names()) {
            hipFunction_t f = nullptr;
            HIP_TRY(hipModuleGetFunction(&f, c->module, name.c_str()));
            c->fn[name] = f;
        }
        HIP_TRY(hipStreamCreate(&c->stream));
        HIP_TRY(hipMalloc((void**)&c->fault_dev, 256));
        HIP_TRY(hipMemsetAsync(c->fault_dev, 0, 256, c->stream));
        HIP_TRY(hipEventCreate(&c->ev0));
        HIP_TRY(hipEventCreate(&c->ev1));
        HIP_TRY(hipStreamSynchronize(c->stream));
        return APK_OK;
    }();
    if (rc != APK_OK) {
        apk_shutdown(c);
        return rc;
    }
    *out = c;
    return APK_OK;
}

int apk_shutdown(apk_ctx* c) {
    if (!c) return APK_OK;
    (void)hipSetDevice(c->device);
    if (c->capturing) {
        hipGraph_t g = nullptr;
        (void)hipStreamEndCapture(c->stream, &g);
        if (g) (void)hipGraphDestroy(g);
        c->capturing = false;
    }
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    for (auto& kv : c->attached) (void)hipFree(kv.second.dev);
    if (c->ids_stage_dev) (void)hipFree(c->ids_stage_dev);
    if (c->ids_stage_host) (void)hipHostFree(c->ids_stage_host);
    if (c->fault_dev) (void)hipFree(c->fault_dev);
    if (c->argmax_scratch) (void)hipFree(c->argmax_scratch);
    if (c->permute_counts) (void)hipFree(c->permute_counts);
    if (c->ev0) (void)hipEventDestroy(c->ev0);
    if (c->ev1) (void)hipEventDestroy(c->ev1);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    if (c->module) (void)hipModuleUnload(c->module);
    delete c;
    return APK_OK;
}

int apk_sync(apk_ctx* c) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_sync: ctx is NULL");
    std::lock_guard<std::mutex> lock(c->mu);
    NOT_WHILE_CAPTURING(c, "apk_sync");
    uint64_t t0 = now_ns();
    hipError_t e = hipStreamSynchronize(c->stream);
    c->wait_ns += now_ns() - t0;
    if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    return APK_OK;
}

void* apk_stream(apk_ctx* c) { return c ? (void*)c->stream : nullptr; }

int apk_stats(apk_ctx* c, uint64_t* calls, uint64_t* dispatches, uint64_t* encode_ns, uint64_t* wait_ns) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_stats: ctx is NULL");
    if (calls) *calls = c->calls;
    if (dispatches) *dispatches = c->dispatches;
    if (encode_ns) *encode_ns = c->encode_ns;
    if (wait_ns) *wait_ns = c->wait_ns;
    return APK_OK;
}

int apk_take_faults(apk_ctx* c, uint32_t* faults) {
    if (!c || !faults) return fail(APK_DECLINE_NULL, "apk_take_faults: NULL argument");
    std::lock_guard<std::mutex> lock(c->mu);
    NOT_WHILE_CAPTURING(c, "apk_take_faults");
    if (int rc = set_device(c)) return rc;
    uint32_t v = 0;
    HIP_TRY(hipMemcpyAsync(&v, c->fault_dev, 4, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(hipStreamSynchronize(c->stream));
    if (v) {
        HIP_TRY(hipMemsetAsync(c->fault_dev, 0, 4, c->stream));
        HIP_TRY(hipStreamSynchronize(c->stream));
    }
    *faults = v;
    return APK_OK;
}

/* ---------------------------------------------------------------- memory */

int apk_malloc(apk_ctx* c, size_t bytes, void** dev_out) {
    if (!c || !dev_out) return fail(APK_DECLINE_NULL, "apk_malloc: NULL argument");
    std::lock_guard<std::mutex> lock(c->mu);
    NOT_WHILE_CAPTURING(c, "apk_malloc");
    if (int rc = set_device(c)) return rc;
    HIP_TRY(hipMalloc(dev_out, bytes ? bytes : 16));
    return APK_OK;
}
int apk_free(apk_ctx* c, void* dev) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_free: ctx is NULL");
    std::lock_guard<std::mutex> lock(c->mu);
    NOT_WHILE_CAPTURING(c, "apk_free");
    if (int rc = set_device(c)) return rc;
    HIP_TRY(hipStreamSynchronize(c->stream));
    HIP_TRY(hipFree(dev));
    return APK_OK;
}
int apk_h2d(apk_ctx* c, void* dev_dst, const void* host_src, size_t bytes) {
    if (!c || (bytes && (!dev_dst || !host_src))) return fail(APK_DECLINE_NULL, "apk_h2d: NULL argument");
    CallScope s(c);
    NOT_WHILE_CAPTURING(c, "apk_h2d");
    if (int rc = set_device(c)) return rc;
    if (bytes) HIP_TRY(hipMemcpyAsync(dev_dst, host_src, bytes, hipMemcpyHostToDevice, c->stream));
    return APK_OK;
}
int apk_d2h(apk_ctx* c, void* host_dst, const void* dev_src, size_t bytes) {
    if (!c || (bytes && (!host_dst || !dev_src))) return fail(APK_DECLINE_NULL, "apk_d2h: NULL argument");
    CallScope s(c);
    NOT_WHILE_CAPTURING(c, "apk_d2h");
    if (int rc = set_device(c)) return rc;
    if (bytes) HIP_TRY(hipMemcpyAsync(host_dst, dev_src, bytes, hipMemcpyDeviceToHost, c->stream));
    return APK_OK;
}

// gpu::attach / detach keep the reference's ownership rules (gpu/cuda/runtime/device.rs:588-621): a mapping is keyed
// by (host address, length) and counts its owners; attaching a range that lies inside an attached mapping succeeds
// without a copy and without a count; the last detach of a key frees the device copy.  A range that overlaps an
// attached mapping without lying inside it is declined (the two copies could name one host address twice).
int apk_attach(apk_ctx* c, const void* host_base, size_t len) {
    if (!c || !host_base || !len) return fail(APK_DECLINE_NULL, "apk_attach: NULL or empty mapping");
    std::lock_guard<std::mutex> lock(c->mu);
    NOT_WHILE_CAPTURING(c, "apk_attach");
    if (int rc = set_device(c)) return rc;
    const uintptr_t b = (uintptr_t)host_base;
    if (b + len < b) return fail(APK_DECLINE_SHAPE, "apk_attach: the range wraps the address space");
    auto same = c->attached.find(b);
    if (same != c->attached.end() && same->second.len == len) {
        same->second.owners++;
        return APK_OK;  // already resident: one more owner
    }
    for (const auto& kv : c->attached) {
        const uintptr_t s0 = kv.first, s1 = kv.first + kv.second.len;
        if (b >= s0 && b + len <= s1) return APK_OK;  // inside an attached mapping: no copy, not counted
        if (b < s1 && s0 < b + len)
            return fail(APK_DECLINE_SHAPE, "apk_attach: [%p, +%zu) overlaps the attached mapping [%p, +%zu) without lying inside it",
                        host_base, len, (void*)s0, kv.second.len);
    }
    void* dev = nullptr;
    HIP_TRY(hipMalloc(&dev, len));
    hipError_t e = hipMemcpy(dev, host_base, len, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(dev);
        return hip_fail(e, "apk_attach: hipMemcpy");
    }
    c->attached[b] = Mapping{dev, len, 1, ++c->clock};
    return APK_OK;
}
// Drops one owner of the mapping attached as exactly (host_base, len); len 0 names whatever mapping starts at
// host_base.  The last owner frees the device copy, after the stream has drained.  A recorded graph bakes in device
// addresses, so the reference drops its graphs at that point (device.rs:604-621: a later attach at the same host
// address must never run on the old copy); here graphs belong to the caller, so every live graph that was recorded
// while this mapping was attached is marked stale instead: apk_graph_launch declines it from then on, and the
// caller records again after attaching the new file.
int apk_detach_range(apk_ctx* c, const void* host_base, size_t len) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_detach: ctx is NULL");
    std::lock_guard<std::mutex> lock(c->mu);
    NOT_WHILE_CAPTURING(c, "apk_detach");
    auto it = c->attached.find((uintptr_t)host_base);
    if (it == c->attached.end() || (len && it->second.len != len))
        return fail(APK_DECLINE_NOT_ATTACHED, "apk_detach: no mapping was attached as [%p, +%zu)", host_base, len);
    if (it->second.owners > 1) {
        it->second.owners--;
        return APK_OK;
    }
    if (int rc = set_device(c)) return rc;
    HIP_TRY(hipStreamSynchronize(c->stream));  // replays in flight included
    for (apk_graph* g : c->live_graphs)
        if (g->born > it->second.serial) g->stale = true;
    HIP_TRY(hipFree(it->second.dev));
    c->attached.erase(it);
    return APK_OK;
}
int apk_detach(apk_ctx* c, const void* host_base) { return apk_detach_range(c, host_base, 0); }
int apk_resolve(apk_ctx* c, const void* host_ptr, size_t len, void** dev_out) {
    if (!c || !dev_out) return fail(APK_DECLINE_NULL, "apk_resolve: NULL argument");
    std::lock_guard<std::mutex> lock(c->mu);
    uintptr_t p = (uintptr_t)host_ptr;
    auto it = c->attached.upper_bound(p);
    if (it != c->attached.begin()) {
        --it;
        if (p >= it->first && p - it->first <= it->second.len && len <= it->second.len - (p - it->first)) {
            *dev_out = (char*)it->second.dev + (p - it->first);
            return APK_OK;
        }
    }
    *dev_out = nullptr;
    return fail(APK_DECLINE_NOT_ATTACHED, "apk_resolve: foreign memory (not inside an attached mapping)");
}
// gpu::is_attached for one mapping: the owners of the mapping attached as exactly (host_base, len); 0: not attached.
int apk_attached_owners(apk_ctx* c, const void* host_base, size_t len, size_t* owners) {
    if (!c || !owners) return fail(APK_DECLINE_NULL, "apk_attached_owners: NULL argument");
    std::lock_guard<std::mutex> lock(c->mu);
    auto it = c->attached.find((uintptr_t)host_base);
    *owners = (it != c->attached.end() && it->second.len == len) ? it->second.owners : 0;
    return APK_OK;
}

int apk_timer_begin(apk_ctx* c) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_timer_begin: ctx is NULL");
    std::lock_guard<std::mutex> lock(c->mu);
    NOT_WHILE_CAPTURING(c, "apk_timer_begin");
    if (int rc = set_device(c)) return rc;
    HIP_TRY(hipEventRecord(c->ev0, c->stream));
    return APK_OK;
}
int apk_timer_end(apk_ctx* c, float* ms_out) {
    if (!c || !ms_out) return fail(APK_DECLINE_NULL, "apk_timer_end: NULL argument");
    std::lock_guard<std::mutex> lock(c->mu);
    NOT_WHILE_CAPTURING(c, "apk_timer_end");
    if (int rc = set_device(c)) return rc;
    HIP_TRY(hipEventRecord(c->ev1, c->stream));
    uint64_t t0 = now_ns();
    HIP_TRY(hipEventSynchronize(c->ev1));
    c->wait_ns += now_ns() - t0;
    HIP_TRY(hipEventElapsedTime(ms_out, c->ev0, c->ev1));
    return APK_OK;
}

/* ------------------------------------------------------- record / replay */

int apk_capture_begin(apk_ctx* c) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_capture_begin: ctx is NULL");
    std::lock_guard<std::mutex> lock(c->mu);
    if (c->capturing) return fail(APK_DECLINE_CAPTURE, "apk_capture_begin: already recording");
    if (int rc = set_device(c)) return rc;
    // relaxed: other threads of the process stay free to allocate (the mode the reference uses)
    HIP_TRY(hipStreamBeginCapture(c->stream, hipStreamCaptureModeRelaxed));
    c->capturing = true;
    c->capture_nodes = 0;
    c->capture_argmax = false;
    c->capture_permute = false;
    return APK_OK;
}

static int end_capture(apk_ctx* c, hipGraph_t* g) {
    *g = nullptr;
    c->capturing = false;
    HIP_TRY(hipStreamEndCapture(c->stream, g));
    return APK_OK;
}

int apk_capture_end(apk_ctx* c, apk_graph** out) {
    if (!c || !out) return fail(APK_DECLINE_NULL, "apk_capture_end: NULL argument");
    *out = nullptr;
    std::lock_guard<std::mutex> lock(c->mu);
    if (!c->capturing) return fail(APK_DECLINE_CAPTURE, "apk_capture_end: not recording");
    if (int rc = set_device(c)) return rc;
    hipGraph_t g = nullptr;
    if (int rc = end_capture(c, &g)) return rc;
    if (!g) return fail(-(int)hipErrorStreamCaptureInvalidated, "apk_capture_end: the recording was invalidated");
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        return hip_fail(e, "hipGraphInstantiate");
    }
    apk_graph* gr = new apk_graph();
    gr->graph = g;
    gr->exec = exec;
    gr->nodes = c->capture_nodes;
    gr->uses_argmax = c->capture_argmax;
    if (gr->uses_argmax) c->graphs_with_argmax++;
    gr->uses_permute = c->capture_permute;
    if (gr->uses_permute) c->graphs_with_permute++;
    gr->born = ++c->clock;
    c->live_graphs.insert(gr);
    *out = gr;
    return APK_OK;
}

int apk_capture_abort(apk_ctx* c) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_capture_abort: ctx is NULL");
    std::lock_guard<std::mutex> lock(c->mu);
    if (!c->capturing) return APK_OK;
    if (int rc = set_device(c)) return rc;
    hipGraph_t g = nullptr;
    const int rc = end_capture(c, &g);
    if (g) (void)hipGraphDestroy(g);
    return rc;
}

int apk_graph_launch(apk_ctx* c, apk_graph* g) {
    if (!c || !g) return fail(APK_DECLINE_NULL, "apk_graph_launch: NULL argument");
    CallScope s(c);
    NOT_WHILE_CAPTURING(c, "apk_graph_launch");
    if (g->stale)
        return fail(APK_DECLINE_NOT_ATTACHED, "apk_graph_launch: a weight mapping that was attached when this graph was recorded has been "
                                              "detached since; the graph holds its old device addresses -- record it again");
    if (int rc = set_device(c)) return rc;
    HIP_TRY(hipGraphLaunch(g->exec, c->stream));
    c->dispatches += g->nodes;
    return APK_OK;
}

int apk_graph_nodes(apk_graph* g, size_t* nodes) {
    if (!g || !nodes) return fail(APK_DECLINE_NULL, "apk_graph_nodes: NULL argument");
    *nodes = g->nodes;
    return APK_OK;
}

int apk_graph_destroy(apk_ctx* c, apk_graph* g) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_graph_destroy: ctx is NULL");
    if (!g) return APK_OK;
    std::lock_guard<std::mutex> lock(c->mu);
    NOT_WHILE_CAPTURING(c, "apk_graph_destroy");
    if (int rc = set_device(c)) return rc;
    HIP_TRY(hipStreamSynchronize(c->stream));  // a replay may still be running
    if (g->uses_argmax && c->graphs_with_argmax) c->graphs_with_argmax--;
    if (g->uses_permute && c->graphs_with_permute) c->graphs_with_permute--;
    c->live_graphs.erase(g);
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
    return APK_OK;
}

/* ------------------------------------------------------------------- ops */

int apk_swiglu(apk_ctx* c, void* gate, const void* up, size_t n, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_swiglu: ctx is NULL");
    CallScope s(c);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_swiglu: dtype %d", dtype);
    if (n == 0) return APK_OK;
    if (!gate || !up) return fail(APK_DECLINE_NULL, "apk_swiglu: NULL tensor");
    if (!aligned16(gate) || !aligned16(up)) return fail(APK_DECLINE_SHAPE, "apk_swiglu: tensors must be 16-byte aligned");
    if (int rc = set_device(c)) return rc;
    const uint64_t vec = 16 / es, nvec = n / vec;
    const unsigned block = stream_block(nvec), per_block = block;  // one 16-byte tile per lane
    uint64_t grid = (nvec + per_block - 1) / per_block;
    if (grid == 0) grid = 1;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_swiglu: n too large");
    uint64_t n64 = n;
    void* args[] = {&gate, &up, &n64};
    return launch_keyed(c, OP_SWIGLU, (uint32_t)dtype, [&] { return std::string(dtype == APK_F32 ? "apk_swiglu_f32" : "apk_swiglu_f16"); },
                        (unsigned)grid, block, 0, args);
}

int apk_geglu_tanh(apk_ctx* c, void* gate, const void* up, size_t n, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_geglu_tanh: ctx is NULL");
    CallScope s(c);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_geglu_tanh: dtype %d", dtype);
    if (n == 0) return APK_OK;
    if (!gate || !up) return fail(APK_DECLINE_NULL, "apk_geglu_tanh: NULL tensor");
    if (!aligned16(gate) || !aligned16(up)) return fail(APK_DECLINE_SHAPE, "apk_geglu_tanh: tensors must be 16-byte aligned");
    if (int rc = set_device(c)) return rc;
    const uint64_t vec = 16 / es, nvec = n / vec;
    const unsigned block = stream_block(nvec), per_block = block;  // one 16-byte tile per lane
    uint64_t grid = (nvec + per_block - 1) / per_block;
    if (grid == 0) grid = 1;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_geglu_tanh: n too large");
    uint64_t n64 = n;
    void* args[] = {&gate, &up, &n64};
    return launch_keyed(c, OP_GEGLU, (uint32_t)dtype, [&] { return std::string(dtype == APK_F32 ? "apk_geglu_tanh_f32" : "apk_geglu_tanh_f16"); },
                        (unsigned)grid, block, 0, args);
}

int apk_add_assign(apk_ctx* c, void* a, const void* b, size_t n, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_add_assign: ctx is NULL");
    CallScope s(c);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_add_assign: dtype %d", dtype);
    if (n == 0) return APK_OK;
    if (!a || !b) return fail(APK_DECLINE_NULL, "apk_add_assign: NULL tensor");
    if (!aligned16(a) || !aligned16(b)) return fail(APK_DECLINE_SHAPE, "apk_add_assign: tensors must be 16-byte aligned");
    if (int rc = set_device(c)) return rc;
    const uint64_t nvec = n / (16 / es);
    const unsigned block = stream_block(nvec);
    uint64_t grid = (nvec + block - 1) / block;
    if (grid == 0) grid = 1;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_add_assign: n too large");
    uint64_t n64 = n;
    void* args[] = {&a, &b, &n64};
    return launch_keyed(c, OP_ADD_ASSIGN, (uint32_t)dtype,
                        [&] { return std::string(dtype == APK_F32 ? "apk_add_assign_f32" : "apk_add_assign_f16"); }, (unsigned)grid, block, 0, args);
}

int apk_add_scaled(apk_ctx* c, void* dst, const void* src, size_t n, float scale, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_add_scaled: ctx is NULL");
    CallScope s(c);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_add_scaled: dtype %d", dtype);
    if (n == 0) return APK_OK;
    if (!dst || !src) return fail(APK_DECLINE_NULL, "apk_add_scaled: NULL tensor");
    if (dst == src) return fail(APK_DECLINE_SHAPE, "apk_add_scaled: dst and src must be two tensors");
    if (!aligned16(dst) || !aligned16(src)) return fail(APK_DECLINE_SHAPE, "apk_add_scaled: tensors must be 16-byte aligned");
    if (int rc = set_device(c)) return rc;
    const uint64_t nvec = n / (16 / es);
    const unsigned block = stream_block(nvec);
    uint64_t grid = (nvec + block - 1) / block;
    if (grid == 0) grid = 1;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_add_scaled: n too large");
    uint64_t n64 = n;
    void* args[] = {&dst, &src, &n64, &scale};
    return launch(c, dtype == APK_F32 ? "apk_add_scaled_f32" : "apk_add_scaled_f16", (unsigned)grid, block, 0, args);
}

int apk_cast(apk_ctx* c, const void* src, int src_dtype, void* dst, int dst_dtype, size_t n) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_cast: ctx is NULL");
    CallScope s(c);
    if (!elem_size(src_dtype) || !elem_size(dst_dtype) || src_dtype == dst_dtype)
        return fail(APK_DECLINE_UNSUPPORTED, "apk_cast: from dtype %d to dtype %d", src_dtype, dst_dtype);
    if (n == 0) return APK_OK;
    if (!src || !dst) return fail(APK_DECLINE_NULL, "apk_cast: NULL tensor");
    if (!aligned16(src) || !aligned16(dst)) return fail(APK_DECLINE_SHAPE, "apk_cast: tensors must be 16-byte aligned");
    if (int rc = set_device(c)) return rc;
    const unsigned block = stream_block(n / 8);
    uint64_t grid = (n / 4 + 2 * block - 1) / (2 * block);  // four elements per lane and step, two steps
    if (grid == 0) grid = 1;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_cast: n too large");
    uint64_t n64 = n;
    void* args[] = {&src, &dst, &n64};
    return launch(c, src_dtype == APK_F32 ? "apk_cast_f32_f16" : "apk_cast_f16_f32", (unsigned)grid, block, 0, args);
}

int apk_softmax_rows(apk_ctx* c, float* x, size_t rows, size_t n) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_softmax_rows: ctx is NULL");
    CallScope s(c);
    if (rows == 0 || n == 0) return APK_OK;
    if (!x) return fail(APK_DECLINE_NULL, "apk_softmax_rows: NULL tensor");
    // the reference sums a row's exponentials one after the other in f32; a parallel sum stays
    // within 1e-5 of that only while rows are short (router widths), so longer rows are declined
    if (n > 4096) return fail(APK_DECLINE_UNSUPPORTED, "apk_softmax_rows: rows of %zu (at most 4096)", n);
    if (rows > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_softmax_rows: too large");
    if (int rc = set_device(c)) return rc;
    int rows_i = (int)rows, n_i = (int)n;
    void* args[] = {&x, &rows_i, &n_i};
    return launch(c, "apk_softmax_rows", (unsigned)((rows + 3) / 4), 256, 0, args);
}

int apk_add_rmsnorm_rows(apk_ctx* c, void* x, const void* delta, void* h, const float* gamma, size_t n, size_t rows,
                         float eps, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_add_rmsnorm_rows: ctx is NULL");
    CallScope s(c);
    if (!elem_size(dtype)) return fail(APK_DECLINE_UNSUPPORTED, "apk_add_rmsnorm_rows: dtype %d", dtype);
    if (rows == 0) return APK_OK;
    if (!x || !h || !gamma) return fail(APK_DECLINE_NULL, "apk_add_rmsnorm_rows: NULL tensor");
    apk_plan p;
    if (int rc = plan_add_rmsnorm(n, rows, dtype, &p)) return rc;
    // the element-wise and the several-rows-per-wave kernels read a row twice: the norm must not land on it
    if (p.variant != ADDNORM_TILED && h == x && delta)
        return fail(APK_DECLINE_SHAPE, "apk_add_rmsnorm_rows: h aliases x while delta is given");
    if (p.variant != ADDNORM_RAGGED && (!aligned16(x) || !aligned16(h) || !aligned16(gamma) || (delta && !aligned16(delta))))
        return fail(APK_DECLINE_SHAPE, "apk_add_rmsnorm_rows: tensors must be 16-byte aligned");
    if (int rc = set_device(c)) return rc;
    int n_i = (int)n;
    uint32_t rows32 = (uint32_t)rows;
    if (p.variant == ADDNORM_RAGGED) {
        void* rargs[] = {&x, &delta, &h, &gamma, &n_i, &eps};
        return launch(c, p.kernel, p.grid, p.block, 0, rargs);
    }
    if (p.variant == ADDNORM_SMALL) {
        void* sargs[] = {&x, &delta, &h, &gamma, &n_i, &rows32, &eps};
        return launch(c, p.kernel, p.grid, p.block, 0, sargs);
    }
    void* args[] = {&x, &delta, &h, &gamma, &n_i, &eps, &p.rows_per_block, &rows32};
    return launch_keyed(c, OP_ADDNORM, (uint32_t)dtype << 8 | p.tiles_per_lane, [&] { return std::string(p.kernel); }, p.grid, p.block, 0,
                        args);
}

int apk_postnorm_add_rmsnorm_rows(apk_ctx* c, void* x, void* delta, const float* post_gamma, void* h, const float* gamma,
                                  size_t n, size_t rows, float eps, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_postnorm_add_rmsnorm_rows: ctx is NULL");
    if (!elem_size(dtype)) return fail(APK_DECLINE_UNSUPPORTED, "apk_postnorm_add_rmsnorm_rows: dtype %d", dtype);
    if (rows == 0) return APK_OK;
    if (!x || !delta || !post_gamma || !h || !gamma) return fail(APK_DECLINE_NULL, "apk_postnorm_add_rmsnorm_rows: NULL tensor");
    if (h == x || h == delta || x == delta) return fail(APK_DECLINE_SHAPE, "apk_postnorm_add_rmsnorm_rows: x, delta and h must be distinct");
    apk_plan p;
    if (int rc = plan_add_rmsnorm(n, rows, dtype, &p, true)) return rc;
    if (p.variant != ADDNORM_TILED) {
        // rows outside the tiled kernels (not whole 16-byte tiles, longer than they hold, short rows in bulk):
        // the reference's own two steps, the delta normalised in place first
        // (the one decline the second step could raise after the first has run is checked first)
        apk_plan p2;
        if (int rc = plan_add_rmsnorm(n, rows, dtype, &p2)) return rc;
        if (p2.variant != ADDNORM_RAGGED && (!aligned16(x) || !aligned16(h) || !aligned16(gamma) || !aligned16(delta) || !aligned16(post_gamma)))
            return fail(APK_DECLINE_SHAPE, "apk_postnorm_add_rmsnorm_rows: tensors must be 16-byte aligned");
        if (int rc = apk_add_rmsnorm_rows(c, delta, nullptr, delta, post_gamma, n, rows, eps, dtype)) return rc;
        return apk_add_rmsnorm_rows(c, x, delta, h, gamma, n, rows, eps, dtype);
    }
    CallScope s(c);
    if (!aligned16(x) || !aligned16(h) || !aligned16(gamma) || !aligned16(delta) || !aligned16(post_gamma))
        return fail(APK_DECLINE_SHAPE, "apk_postnorm_add_rmsnorm_rows: tensors must be 16-byte aligned");
    if (int rc = set_device(c)) return rc;
    int n_i = (int)n;
    uint32_t rows32 = (uint32_t)rows;
    void* args[] = {&x, &delta, &h, &gamma, &n_i, &eps, &p.rows_per_block, &rows32, &post_gamma};
    return launch(c, p.kernel, p.grid, p.block, 0, args);
}

struct QkvBias {  // the projection biases of apk_attn_prologue_rows (f32; any of them NULL: none for that tensor)
    const float* q = nullptr;
    const float* k = nullptr;
    const float* v = nullptr;  // only with the cache store: added to v in place and to the cached row
};

struct KvStore {  // the fused K/V cache store of apk_qknorm_rope_kv_store (all NULL/0: plain op)
    const void* v = nullptr;
    const uint32_t* cache_pos = nullptr;
    void* k_cache = nullptr;
    void* v_cache = nullptr;
    size_t capacity = 0;
};

// style: 0 = NeoX pairs (i, i + rot_dim/2), 1 = adjacent pairs (2i, 2i+1).  validate_only: every
// check, no launch (so a caller that chains two ops can decline before the first one runs).
static int qknorm_rope_common(apk_ctx* c, void* q, void* k, const float* qw, const float* kw, const float* rope, size_t rows,
                              size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, float eps, int dtype,
                              const KvStore* kv, int style = 0, bool validate_only = false, const QkvBias* bias = nullptr) {
    apk_plan p;
    if (bias && !bias->q && !bias->k && !bias->v) bias = nullptr;
    const bool with_norm = qw || kw;
    if (int rc = plan_qknorm_rope(rows, n_q, n_kv, head_dim, rot_dim, style, dtype, kv != nullptr, &p, bias != nullptr, with_norm)) return rc;
    if (rows == 0 || n_q + n_kv == 0) return APK_OK;
    if ((n_q && !q) || (n_kv && !k) || (!rope && rot_dim)) return fail(APK_DECLINE_NULL, "apk_qknorm_rope: NULL tensor");
    if ((q && !aligned16(q)) || (k && !aligned16(k)) || !aligned16(rope) || (qw && !aligned16(qw)) || (kw && !aligned16(kw)))
        return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope: tensors must be 16-byte aligned");
    if (kv) {
        if (!kv->v || !kv->cache_pos || !kv->k_cache || !kv->v_cache) return fail(APK_DECLINE_NULL, "apk_qknorm_rope_kv_store: NULL tensor");
        if (!aligned16(kv->v) || !aligned16(kv->k_cache) || !aligned16(kv->v_cache))
            return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope_kv_store: tensors must be 16-byte aligned");
        if (kv->capacity == 0 || kv->capacity > 0xffffffffu) return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope_kv_store: capacity");
    }
    QkvBias nb;
    if (bias) {
        nb = *bias;
        if ((nb.q && !aligned16(nb.q)) || (nb.k && !aligned16(nb.k)) || (nb.v && !aligned16(nb.v)))
            return fail(APK_DECLINE_SHAPE, "apk_attn_prologue_rows: biases must be 16-byte aligned");
        if (nb.v && !kv) return fail(APK_DECLINE_SHAPE, "apk_attn_prologue_rows: v_bias rides on the cache store here");
    }
    if (validate_only) return APK_OK;
    if (int rc = set_device(c)) return rc;
    int rows_i = (int)rows, nq_i = (int)n_q, nkv_i = (int)n_kv, rot_i = (int)rot_dim;
    if (p.variant == QK_GENERIC) {
        int hd_i = (int)head_dim, half_i = (int)(rot_dim / 2);
        void* gargs[] = {&q, &k, &qw, &kw, &rope, &rows_i, &nq_i, &nkv_i, &hd_i, &half_i, &style, &eps, &nb.q, &nb.k};
        return launch(c, p.kernel, p.grid, p.block, 0, gargs);
    }
    auto which = [&] { return std::string(p.kernel); };
    const uint32_t variant = (uint32_t)with_norm << 22 | (uint32_t)(bias != nullptr) << 21 | (uint32_t)style << 20 | (uint32_t)dtype << 16 | (uint32_t)head_dim << 4 | p.tiles_per_lane;
    if (kv && bias) {
        uint32_t cap32 = (uint32_t)kv->capacity;
        void* kargs[] = {&q, &k, (void*)&kv->v, &qw, &kw, &rope, (void*)&kv->cache_pos, (void*)&kv->k_cache, (void*)&kv->v_cache,
                         &cap32, &rows_i, &nq_i, &nkv_i, &eps, &c->fault_dev, &rot_i, &nb.q, &nb.k, &nb.v};
        return launch_keyed(c, OP_QKROPE_KV, variant, which, p.grid, p.block, 0, kargs);
    }
    if (bias) {
        void* bargs[] = {&q, &k, &qw, &kw, &rope, &rows_i, &nq_i, &nkv_i, &eps, &rot_i, &nb.q, &nb.k};
        return launch_keyed(c, OP_QKROPE, variant, which, p.grid, p.block, 0, bargs);
    }
    if (kv) {
        uint32_t cap32 = (uint32_t)kv->capacity;
        void* kargs[] = {&q, &k, (void*)&kv->v, &qw, &kw, &rope, (void*)&kv->cache_pos, (void*)&kv->k_cache, (void*)&kv->v_cache,
                         &cap32, &rows_i, &nq_i, &nkv_i, &eps, &c->fault_dev, &rot_i};
        return launch_keyed(c, OP_QKROPE_KV, variant, which, p.grid, p.block, 0, kargs);
    }
    void* args[] = {&q, &k, &qw, &kw, &rope, &rows_i, &nq_i, &nkv_i, &eps, &rot_i};
    return launch_keyed(c, OP_QKROPE, variant, which, p.grid, p.block, 0, args);
}

int apk_qknorm_rope_neox(apk_ctx* c, void* q, void* k, const float* qw, const float* kw, const float* rope,
                         size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, float eps, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_qknorm_rope_neox: ctx is NULL");
    CallScope s(c);
    return qknorm_rope_common(c, q, k, qw, kw, rope, rows, n_q, n_kv, head_dim, rot_dim, eps, dtype, nullptr, 0);
}

int apk_qknorm_rope_norm(apk_ctx* c, void* q, void* k, const float* qw, const float* kw, const float* rope,
                         size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, float eps, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_qknorm_rope_norm: ctx is NULL");
    CallScope s(c);
    return qknorm_rope_common(c, q, k, qw, kw, rope, rows, n_q, n_kv, head_dim, rot_dim, eps, dtype, nullptr, 1);
}

int apk_qknorm_rope_pos(apk_ctx* c, void* q, void* k, const void* v, const float* qw, const float* kw, const uint32_t* positions,
                        const float* inv_freq, void* k_cache, void* v_cache, size_t capacity, size_t rows, size_t n_q,
                        size_t n_kv, size_t head_dim, size_t rot_dim, int adjacent_pairs, float eps, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_qknorm_rope_pos: ctx is NULL");
    CallScope s(c);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_qknorm_rope_pos: dtype %d", dtype);
    if (head_dim == 0 || head_dim > 65536 || rot_dim % 2 || rot_dim > head_dim)
        return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope_pos: head_dim %zu, rot_dim %zu", head_dim, rot_dim);
    if (rows > 64)
        return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope_pos: %zu rows (a decode-sized batch of at most 64; beyond that build the table "
                                       "with apk_rope_table)", rows);
    if (n_q > 65535 || n_kv > 65535) return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope_pos: too many heads");
    const bool store = k_cache || v_cache;
    if (store && (!k_cache || !v_cache || !v)) return fail(APK_DECLINE_NULL, "apk_qknorm_rope_pos: the cache store needs v, k_cache and v_cache");
    if (store && n_kv == 0) return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope_pos: no k heads to store");
    if (store && (capacity == 0 || capacity > 0xffffffffu)) return fail(APK_DECLINE_SHAPE, "apk_qknorm_rope_pos: capacity");
    if (rows == 0 || n_q + n_kv == 0) return APK_OK;
    if ((n_q && !q) || (n_kv && !k) || !positions || (rot_dim && !inv_freq)) return fail(APK_DECLINE_NULL, "apk_qknorm_rope_pos: NULL tensor");
    if (int rc = set_device(c)) return rc;
    int rows_i = (int)rows, nq_i = (int)n_q, nkv_i = (int)n_kv, hd_i = (int)head_dim, half_i = (int)(rot_dim / 2), style = adjacent_pairs ? 1 : 0;
    uint32_t cap32 = (uint32_t)capacity;
    void* args[] = {&q, &k, &v, &qw, &kw, &positions, &inv_freq, &k_cache, &v_cache, &cap32, &rows_i, &nq_i, &nkv_i, &hd_i, &half_i, &style,
                    &eps, &c->fault_dev};
    const uint64_t waves = (uint64_t)rows * (n_q + n_kv + (store ? n_kv : 0));
    return launch(c, dtype == APK_F32 ? "apk_qknorm_rope_pos_f32" : "apk_qknorm_rope_pos_f16", (unsigned)((waves + 3) / 4), 256, 0, args);
}

int apk_qknorm_rope_kv_store(apk_ctx* c, void* q, void* k, const void* v, const float* qw, const float* kw,
                             const float* rope, const uint32_t* cache_pos, void* k_cache, void* v_cache, size_t capacity,
                             size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, float eps, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_qknorm_rope_kv_store: ctx is NULL");
    CallScope s(c);
    KvStore kv;
    kv.v = v; kv.cache_pos = cache_pos; kv.k_cache = k_cache; kv.v_cache = v_cache; kv.capacity = capacity;
    return qknorm_rope_common(c, q, k, qw, kw, rope, rows, n_q, n_kv, head_dim, rot_dim, eps, dtype, &kv);
}

int apk_qknorm_rope_norm_kv_store(apk_ctx* c, void* q, void* k, const void* v, const float* qw, const float* kw,
                                  const float* rope, const uint32_t* cache_pos, void* k_cache, void* v_cache, size_t capacity,
                                  size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, float eps, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_qknorm_rope_norm_kv_store: ctx is NULL");
    CallScope s(c);
    KvStore kv;
    kv.v = v; kv.cache_pos = cache_pos; kv.k_cache = k_cache; kv.v_cache = v_cache; kv.capacity = capacity;
    return qknorm_rope_common(c, q, k, qw, kw, rope, rows, n_q, n_kv, head_dim, rot_dim, eps, dtype, &kv, 1);
}

// the caller holds the context (CallScope)
static int add_bias_rows_locked(apk_ctx* c, void* x, const float* bias, size_t rows, size_t n, int dtype) {
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_add_bias_rows: dtype %d", dtype);
    if (rows == 0 || n == 0) return APK_OK;
    if (!x || !bias) return fail(APK_DECLINE_NULL, "apk_add_bias_rows: NULL tensor");
    if (!aligned16(x) || !aligned16(bias)) return fail(APK_DECLINE_SHAPE, "apk_add_bias_rows: tensors must be 16-byte aligned");
    if (n > 0xffffffffu || rows > ((uint64_t)1 << 40) / n) return fail(APK_DECLINE_SHAPE, "apk_add_bias_rows: sizes out of range");
    if (int rc = set_device(c)) return rc;
    const size_t vec = 16 / es;
    const uint64_t lanes = n % vec == 0 ? (uint64_t)rows * (n / vec) : (uint64_t)rows * n;
    const unsigned block = stream_block(lanes);
    const uint64_t grid = (lanes + block - 1) / block;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_add_bias_rows: too large");
    uint64_t rows64 = rows;
    uint32_t n32 = (uint32_t)n;
    void* args[] = {&x, &bias, &rows64, &n32};
    return launch(c, dtype == APK_F32 ? "apk_add_bias_rows_f32" : "apk_add_bias_rows_f16", (unsigned)grid, block, 0, args);
}

int apk_add_bias_rows(apk_ctx* c, void* x, const float* bias, size_t rows, size_t n, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_add_bias_rows: ctx is NULL");
    CallScope s(c);
    return add_bias_rows_locked(c, x, bias, rows, n, dtype);
}

int apk_attn_prologue_rows(apk_ctx* c, const apk_attn_prologue* a) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_attn_prologue_rows: ctx is NULL");
    if (!a) return fail(APK_DECLINE_NULL, "apk_attn_prologue_rows: args is NULL");
    CallScope s(c);
    const bool store = a->k_cache || a->v_cache || a->cache_pos;
    KvStore kv;
    kv.v = a->v; kv.cache_pos = a->cache_pos; kv.k_cache = a->k_cache; kv.v_cache = a->v_cache; kv.capacity = a->capacity;
    QkvBias bias;
    bias.q = a->q_bias; bias.k = a->k_bias;
    bias.v = store ? a->v_bias : nullptr;
    const int style = a->adjacent_pairs ? 1 : 0;
    if (a->v_bias && !store && a->rows && a->n_kv) {
        // no cache store: v is not read by the q/k kernel, its bias is a launch of its own -- after every check of
        // the main op, so that a decline leaves v as it was
        if (int rc = qknorm_rope_common(c, a->q, a->k, a->q_norm, a->k_norm, a->rope, a->rows, a->n_q, a->n_kv, a->head_dim, a->rot_dim,
                                        a->eps, a->dtype, nullptr, style, true, &bias))
            return rc;
        if (!a->v) return fail(APK_DECLINE_NULL, "apk_attn_prologue_rows: v_bias without v");
        if (int rc = add_bias_rows_locked(c, a->v, a->v_bias, a->rows, a->n_kv * a->head_dim, a->dtype)) return rc;
    }
    return qknorm_rope_common(c, a->q, a->k, a->q_norm, a->k_norm, a->rope, a->rows, a->n_q, a->n_kv, a->head_dim, a->rot_dim, a->eps,
                              a->dtype, store ? &kv : nullptr, style, false, &bias);
}

int apk_layer_prologue(apk_ctx* c, void* x, const void* delta, void* h, const float* gamma, size_t n, void* q, void* k,
                       const float* qw, const float* kw, const float* rope, size_t rows, size_t n_q, size_t n_kv,
                       size_t head_dim, size_t rot_dim, float eps, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_layer_prologue: ctx is NULL");
    const int es = elem_size(dtype);
    bool fused = es != 0 && rows > 0 && n_q + n_kv > 0 && n > 0 && x && h && gamma && rope && (!n_q || q) && (!n_kv || k) &&
                 (head_dim == 64 || head_dim == 128 || head_dim == 256) && rot_dim == head_dim;
    size_t threads = 0;
    if (fused) {
        const size_t vec = 16 / es, nchunks = n / vec;
        threads = (nchunks + 63) / 64 * 64;  // one 16-byte tile per lane
        fused = n % vec == 0 && threads <= 1024 && rows * (threads / 64) <= 2048 && rows <= 0x7fffffffu &&
                aligned16(x) && aligned16(h) && aligned16(gamma) && (!delta || aligned16(delta)) && (!q || aligned16(q)) &&
                (!k || aligned16(k)) && aligned16(rope) && (!qw || aligned16(qw)) && (!kw || aligned16(kw)) &&
                n_q <= 65535 && n_kv <= 65535;
    }
    if (!fused) {
        // outside the single-launch shape (large batches are bandwidth-bound, not launch-bound):
        // the same result as two launches; every check and decline is theirs
        // (the second op is validated before the first runs: a decline leaves nothing half done)
        if (int rc = qknorm_rope_common(c, q, k, qw, kw, rope, rows, n_q, n_kv, head_dim, rot_dim, eps, dtype, nullptr, 0, true))
            return rc;
        if (int rc = apk_add_rmsnorm_rows(c, x, delta, h, gamma, n, rows, eps, dtype)) return rc;
        return apk_qknorm_rope_neox(c, q, k, qw, kw, rope, rows, n_q, n_kv, head_dim, rot_dim, eps, dtype);
    }
    CallScope s(c);
    if (int rc = set_device(c)) return rc;
    const size_t epl = 16 / es, lph = head_dim / 2 / epl, hpw = 64 / lph;
    const uint64_t qk_waves = (uint64_t)rows * ((n_q + hpw - 1) / hpw + (n_kv + hpw - 1) / hpw);
    const uint64_t wpb = threads / 64;
    const uint64_t grid = rows + (qk_waves + wpb - 1) / wpb;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_layer_prologue: too large");
    int n_i = (int)n, rows_i = (int)rows, nq_i = (int)n_q, nkv_i = (int)n_kv;
    void* args[] = {&x, &delta, &h, &gamma, &n_i, &q, &k, &qw, &kw, &rope, &rows_i, &nq_i, &nkv_i, &eps};
    return launch_keyed(c, OP_PROLOGUE, (uint32_t)dtype << 16 | (uint32_t)head_dim,
                        [&] { return std::string("apk_layer_prologue_") + (dtype == APK_F32 ? "f32" : "f16") + "_hd" + std::to_string(head_dim); },
                        (unsigned)grid, (unsigned)threads, 0, args);
}

int apk_rope_inv_freq(size_t rot_dim, float base, float* inv_freq) {
    if (rot_dim >= 2 && !inv_freq) return fail(APK_DECLINE_NULL, "apk_rope_inv_freq: inv_freq is NULL");
    for (size_t i = 0; i < rot_dim / 2; i++) inv_freq[i] = powf(base, -2.0f * (float)i / (float)rot_dim);
    return APK_OK;
}

int apk_rope_table(apk_ctx* c, const uint32_t* positions, const float* inv_freq, size_t rows, size_t half, float* table) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_rope_table: ctx is NULL");
    CallScope s(c);
    if (rows == 0 || half == 0) return APK_OK;
    if (!positions || !inv_freq || !table) return fail(APK_DECLINE_NULL, "apk_rope_table: NULL tensor");
    if (rows > 0x7fffffffu || half > 0x7fffffffu || rows * half > 0x7fffffffull * 256)
        return fail(APK_DECLINE_SHAPE, "apk_rope_table: too large");
    if (int rc = set_device(c)) return rc;
    int rows_i = (int)rows, half_i = (int)half;
    const uint64_t grid = ((uint64_t)rows * half + 255) / 256;
    void* args[] = {&positions, &inv_freq, &rows_i, &half_i, &table};
    return launch(c, "apk_rope_table", (unsigned)grid, 256, 0, args);
}

// ids_dev == nullptr with have_ids == false: the rows row0, row0 + 1, ... (apk_dequant_rows)
static int embed_common(apk_ctx* c, int fmt, const void* table, size_t vocab, size_t n_in, const uint32_t* ids_dev,
                        size_t t, void* out, int out_dtype, float scale = 1.0f, bool have_ids = true, uint32_t row0 = 0) {
    apk_plan p;
    if (int rc = plan_embed(fmt, n_in, t, out_dtype, &p)) return rc;
    if (t == 0) return APK_OK;
    if (!table || (have_ids && !ids_dev) || !out) return fail(APK_DECLINE_NULL, "apk_embed_rows: NULL tensor");
    if (!aligned16(table) || !aligned16(out)) return fail(APK_DECLINE_SHAPE, "apk_embed_rows: table/out must be 16-byte aligned");
    if (vocab == 0 || vocab > 0xffffffffu) return fail(APK_DECLINE_SHAPE, "apk_embed_rows: sizes out of range");
    if (int rc = set_device(c)) return rc;
    uint32_t vocab32 = (uint32_t)vocab;
    int n_i = (int)n_in;
    const uint32_t key = (uint32_t)fmt << 8 | (uint32_t)out_dtype;
    auto which = [&] { return std::string(p.kernel); };
    if (p.variant == EMBED_Q4K) {
        void* args[] = {&table, &vocab32, &n_i, &ids_dev, &out, &c->fault_dev, &scale, &row0};
        return launch_keyed(c, OP_EMBED, key, which, p.grid, p.block, 0, args);
    }
    if (p.variant == EMBED_STAGED) {
        uint64_t table_bytes = (uint64_t)vocab * apk_row_bytes(fmt, n_in);
        void* args[] = {&table, &table_bytes, &vocab32, &n_i, &ids_dev, &out, &c->fault_dev, &scale, &row0};
        return launch_keyed(c, OP_EMBED, key, which, p.grid, p.block, p.shmem, args);
    }
    uint32_t rows32 = (uint32_t)t;  // the super-block kernels number their lanes across the batch; the others slice a row
    void* args[] = {&table, &vocab32, &n_i, &ids_dev, p.variant == EMBED_SUPERBLOCK ? (void*)&rows32 : (void*)&p.slices_per_row, &out,
                    &c->fault_dev, &scale, &row0};
    return launch_keyed(c, OP_EMBED, key, which, p.grid, p.block, 0, args);
}

int apk_embed_rows(apk_ctx* c, int fmt, const void* table, size_t vocab, size_t n_in, const uint32_t* ids, size_t t,
                   void* out, int out_dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_embed_rows: ctx is NULL");
    CallScope s(c);
    return embed_common(c, fmt, table, vocab, n_in, ids, t, out, out_dtype);
}

int apk_embed_rows_scaled(apk_ctx* c, int fmt, const void* table, size_t vocab, size_t n_in, const uint32_t* ids, size_t t,
                          float scale, void* out, int out_dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_embed_rows_scaled: ctx is NULL");
    CallScope s(c);
    return embed_common(c, fmt, table, vocab, n_in, ids, t, out, out_dtype, scale);
}

int apk_dequant_rows(apk_ctx* c, int fmt, const void* table, size_t n_rows, size_t n_in, size_t row0, size_t count,
                     void* out, int out_dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_dequant_rows: ctx is NULL");
    CallScope s(c);
    if (row0 > n_rows || count > n_rows - row0)
        return fail(APK_DECLINE_RANGE, "apk_dequant_rows: rows [%zu, +%zu) of %zu", row0, count, n_rows);
    return embed_common(c, fmt, table, n_rows, n_in, nullptr, count, out, out_dtype, 1.0f, false, (uint32_t)row0);
}

int apk_embed_rows_host_ids(apk_ctx* c, int fmt, const void* table, size_t vocab, size_t n_in,
                            const uint32_t* ids_host, size_t t, void* out, int out_dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_embed_rows_host_ids: ctx is NULL");
    CallScope s(c);
    NOT_WHILE_CAPTURING(c, "apk_embed_rows_host_ids");
    if (t == 0) return APK_OK;
    if (!ids_host) return fail(APK_DECLINE_NULL, "apk_embed_rows_host_ids: ids is NULL");
    for (size_t i = 0; i < t; i++)
        if (ids_host[i] >= vocab)
            return fail(APK_DECLINE_RANGE, "apk_embed_rows_host_ids: token %u at %zu >= vocab %zu", ids_host[i], i, vocab);
    // a single token (a decode step with the sampler on the host): the id travels as a kernel argument, with no
    // staging copy and no wait on the stream
    if (t == 1) return embed_common(c, fmt, table, vocab, n_in, nullptr, 1, out, out_dtype, 1.0f, false, ids_host[0]);
    if (int rc = set_device(c)) return rc;
    if (t > c->ids_stage_cap) {
        // the previous staging buffer may still be read by an enqueued copy
        HIP_TRY(hipStreamSynchronize(c->stream));
        if (c->ids_stage_dev) (void)hipFree(c->ids_stage_dev);
        if (c->ids_stage_host) (void)hipHostFree(c->ids_stage_host);
        c->ids_stage_dev = nullptr;
        c->ids_stage_host = nullptr;
        c->ids_stage_cap = 0;
        size_t cap = t < 4096 ? 4096 : t;
        HIP_TRY(hipHostMalloc((void**)&c->ids_stage_host, cap * 4, hipHostMallocDefault));
        HIP_TRY(hipMalloc((void**)&c->ids_stage_dev, cap * 4));
        c->ids_stage_cap = cap;
    } else {
        // the pinned buffer is reused: wait until the previous copy out of it has run
        HIP_TRY(hipStreamSynchronize(c->stream));
    }
    memcpy(c->ids_stage_host, ids_host, t * 4);
    HIP_TRY(hipMemcpyAsync(c->ids_stage_dev, c->ids_stage_host, t * 4, hipMemcpyHostToDevice, c->stream));
    return embed_common(c, fmt, table, vocab, n_in, c->ids_stage_dev, t, out, out_dtype);
}

int apk_route_topk(apk_ctx* c, const float* logits, const float* bias, size_t rows, size_t n_expert, size_t k, int norm,
                   float scale, int sigmoid, uint32_t* ids, float* w) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_route_topk: ctx is NULL");
    CallScope s(c);
    if (n_expert == 0 || n_expert > 1024) return fail(APK_DECLINE_UNSUPPORTED, "apk_route_topk: n_expert %zu (1..1024)", n_expert);
    if (k == 0 || k > n_expert || k > 64) return fail(APK_DECLINE_UNSUPPORTED, "apk_route_topk: k %zu", k);
    if (rows == 0) return APK_OK;
    if (!logits || !ids || !w) return fail(APK_DECLINE_NULL, "apk_route_topk: NULL tensor");
    if (rows > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_route_topk: too large");
    if (int rc = set_device(c)) return rc;
    int rows_i = (int)rows, ne_i = (int)n_expert, k_i = (int)k;
    const unsigned block = 256, per_block = block / 64;
    const uint64_t grid = (rows + per_block - 1) / per_block;
    void* args[] = {&logits, &bias, &rows_i, &ne_i, &k_i, &norm, &scale, &sigmoid, &ids, &w};
    const char* which = n_expert <= 64 ? "apk_route_topk_e64" : n_expert <= 128 ? "apk_route_topk_e128" : n_expert <= 256 ? "apk_route_topk" : "apk_route_topk_wide";
    return launch(c, which, (unsigned)grid, block, 0, args);
}

int apk_moe_permute(apk_ctx* c, const uint32_t* ids, const float* w, size_t rows, size_t k, size_t n_expert,
                    uint32_t* table, uint32_t* n_used, uint32_t* tok, uint32_t* tok_off, uint32_t* hit_row, float* hit_w) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_moe_permute: ctx is NULL");
    CallScope s(c);
    if (n_expert == 0 || n_expert > 1024) return fail(APK_DECLINE_UNSUPPORTED, "apk_moe_permute: n_expert %zu (1..1024)", n_expert);
    if (k == 0 || k > n_expert) return fail(APK_DECLINE_UNSUPPORTED, "apk_moe_permute: k %zu", k);
    if (!table || !n_used || !tok_off) return fail(APK_DECLINE_NULL, "apk_moe_permute: NULL tensor");
    if (rows && (!ids || !w || !tok || !hit_row || !hit_w)) return fail(APK_DECLINE_NULL, "apk_moe_permute: NULL tensor");
    if (rows * k >= 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_moe_permute: rows*k too large");
    if (int rc = set_device(c)) return rc;
    int rows_i = (int)rows, k_i = (int)k, ne_i = (int)n_expert;
    if (rows <= 2048) {
        // one launch: every workgroup (one per expert) walks all picks -- fastest for decode and
        // medium prefill batches
        void* args[] = {&ids, &w, &rows_i, &k_i, &ne_i, &table, &n_used, &tok, &tok_off, &hit_row, &hit_w, &c->fault_dev};
        return launch(c, "apk_moe_permute", (unsigned)n_expert, 512, 0, args);
    }
    // large batches: histogram per part of 1024 tokens, then one workgroup per (expert, part)
    const size_t parts = (rows + 1023) / 1024;
    if (n_expert * parts > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_moe_permute: too large");
    const size_t need = parts * n_expert;
    if (need > c->permute_counts_cap) {
        if (c->capturing || c->graphs_with_permute)
            return fail(APK_DECLINE_CAPTURE, "apk_moe_permute: the scratch would have to grow %s",
                        c->capturing ? "inside a recording (run once unrecorded first)"
                                     : "while a recorded graph holds its address (destroy the graph first)");
        HIP_TRY(hipStreamSynchronize(c->stream));  // a previous launch may still use the old scratch
        if (c->permute_counts) (void)hipFree(c->permute_counts);
        c->permute_counts = nullptr;
        c->permute_counts_cap = 0;
        HIP_TRY(hipMalloc((void**)&c->permute_counts, need * 4));
        c->permute_counts_cap = need;
    }
    if (c->capturing) c->capture_permute = true;
    int parts_i = (int)parts;
    void* cargs[] = {&ids, &rows_i, &k_i, &ne_i, &c->permute_counts, &c->fault_dev};
    if (int rc = launch(c, "apk_moe_count", (unsigned)parts, 512, 0, cargs)) return rc;
    void* rargs[] = {&ids, &w, &rows_i, &k_i, &ne_i, &parts_i, &c->permute_counts, &table, &n_used, &tok, &tok_off, &hit_row, &hit_w};
    return launch(c, "apk_moe_rank", (unsigned)(n_expert * parts), 512, 0, rargs);
}

int apk_route_group(apk_ctx* c, const float* logits, const float* bias, size_t rows, size_t n_expert, size_t k, int norm,
                    float scale, int sigmoid, uint32_t* ids, float* w, uint32_t* table, uint32_t* n_used, uint32_t* tok,
                    uint32_t* tok_off, uint32_t* hit_row, float* hit_w) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_route_group: ctx is NULL");
    if (n_expert == 0 || n_expert > 1024) return fail(APK_DECLINE_UNSUPPORTED, "apk_route_group: n_expert %zu (1..1024)", n_expert);
    if (k == 0 || k > n_expert || k > 64) return fail(APK_DECLINE_UNSUPPORTED, "apk_route_group: k %zu", k);
    if (!table || !n_used || !tok_off) return fail(APK_DECLINE_NULL, "apk_route_group: NULL tensor");
    if (rows && (!logits || !ids || !w || !tok || !hit_row || !hit_w)) return fail(APK_DECLINE_NULL, "apk_route_group: NULL tensor");
    if (rows == 0 || rows > 16) {
        // beyond a decode-sized batch the two launches are bound by their work, not by the launch:
        // the same results from the two entries.  What the second could still decline after the first has
        // run -- its scratch having to grow inside a recording or under a recorded graph -- is checked first.
        if (rows > 2048) {
            std::lock_guard<std::mutex> lock(c->mu);
            if ((rows + 1023) / 1024 * n_expert > c->permute_counts_cap && (c->capturing || c->graphs_with_permute))
                return fail(APK_DECLINE_CAPTURE, "apk_route_group: the grouping scratch would have to grow %s",
                            c->capturing ? "inside a recording (run once unrecorded first)"
                                         : "while a recorded graph holds its address (destroy the graph first)");
        }
        if (int rc = apk_route_topk(c, logits, bias, rows, n_expert, k, norm, scale, sigmoid, ids, w)) return rc;
        return apk_moe_permute(c, ids, w, rows, k, n_expert, table, n_used, tok, tok_off, hit_row, hit_w);
    }
    CallScope s(c);
    if (int rc = set_device(c)) return rc;
    int rows_i = (int)rows, ne_i = (int)n_expert, k_i = (int)k;
    void* args[] = {&logits, &bias, &rows_i, &ne_i, &k_i, &norm, &scale, &sigmoid, &ids, &w, &table, &n_used, &tok, &tok_off, &hit_row, &hit_w};
    const char* which = n_expert <= 64 ? "apk_route_group_small_e64" : n_expert <= 128 ? "apk_route_group_small_e128"
                      : n_expert <= 256 ? "apk_route_group_small_e256" : "apk_route_group_small_e1024";
    return launch(c, which, 1, 1024, 0, args);
}

int apk_gather_rows(apk_ctx* c, const void* src, const uint32_t* tok, size_t src_rows, size_t total_rows, size_t cols,
                    void* dst, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_gather_rows: ctx is NULL");
    CallScope s(c);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_gather_rows: dtype %d", dtype);
    if (total_rows == 0 || cols == 0) return APK_OK;
    if (!src || !tok || !dst) return fail(APK_DECLINE_NULL, "apk_gather_rows: NULL tensor");
    if ((cols * es) % 16 || !aligned16(src) || !aligned16(dst))
        return fail(APK_DECLINE_SHAPE, "apk_gather_rows: rows must be whole 16-byte tiles");
    if (total_rows > 0x7fffffffu || src_rows > 0xffffffffu || cols * es / 16 > 0x7fffffffu)
        return fail(APK_DECLINE_SHAPE, "apk_gather_rows: too large");
    if (int rc = set_device(c)) return rc;
    uint32_t src_rows32 = (uint32_t)src_rows;
    int row_vecs = (int)(cols * es / 16);
    uint32_t total32 = (uint32_t)total_rows;
    void* args[] = {&src, &tok, &src_rows32, &total32, &row_vecs, &dst, &c->fault_dev};
    // groups of 32 destination rows, eight workgroups per group (one per XCD)
    const uint64_t grid = (total_rows + 31) / 32 * 8;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_gather_rows: too large");
    return launch(c, "apk_gather_rows", (unsigned)grid, 256, 0, args);
}

int apk_scatter_rows(apk_ctx* c, const void* src, const uint32_t* hit_row, size_t rows, size_t k, size_t total_rows,
                     size_t cols, void* dst, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_scatter_rows: ctx is NULL");
    CallScope s(c);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_scatter_rows: dtype %d", dtype);
    if (rows == 0 || k == 0 || cols == 0) return APK_OK;
    if (!src || !hit_row || !dst) return fail(APK_DECLINE_NULL, "apk_scatter_rows: NULL tensor");
    if (!aligned16(src) || !aligned16(dst)) return fail(APK_DECLINE_SHAPE, "apk_scatter_rows: rows must be whole 16-byte tiles");
    if (total_rows > 0xffffffffu) return fail(APK_DECLINE_SHAPE, "apk_scatter_rows: too large");
    apk_plan p;
    if (int rc = plan_scatter(rows, k, cols, dtype, &p)) return rc;
    if (int rc = set_device(c)) return rc;
    int row_vecs = (int)(cols * es / 16);
    uint32_t k32 = (uint32_t)k, total32 = (uint32_t)total_rows;
    void* args[] = {&src, &hit_row, &k32, &total32, &row_vecs, &dst, &c->fault_dev, &p.items, &p.slices_per_row};
    return launch(c, p.kernel, p.grid, p.block, 0, args);
}

int apk_moe_shared_hits(apk_ctx* c, const uint32_t* tok_off, const uint32_t* hit_row, const float* hit_w, size_t rows,
                        size_t total_rows, uint32_t* tok_off_out, uint32_t* hit_row_out, float* hit_w_out) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_moe_shared_hits: ctx is NULL");
    CallScope s(c);
    if (!tok_off || !tok_off_out || (rows && (!hit_row_out || !hit_w_out || !hit_row || !hit_w)))
        return fail(APK_DECLINE_NULL, "apk_moe_shared_hits: NULL tensor");
    if (rows >= 0x7fffffffu || total_rows + rows > 0xffffffffu) return fail(APK_DECLINE_SHAPE, "apk_moe_shared_hits: too large");
    if (tok_off_out == tok_off || hit_row_out == hit_row || hit_w_out == hit_w)
        return fail(APK_DECLINE_SHAPE, "apk_moe_shared_hits: the lengthened lists need arrays of their own");
    if (int rc = set_device(c)) return rc;
    uint32_t rows32 = (uint32_t)rows, total32 = (uint32_t)total_rows;
    void* args[] = {&tok_off, &hit_row, &hit_w, &rows32, &total32, &tok_off_out, &hit_row_out, &hit_w_out};
    return launch(c, "apk_moe_shared_hits", (unsigned)((rows + 1 + 255) / 256), 256, 0, args);
}

int apk_moe_combine_add_rmsnorm(apk_ctx* c, void* x, const void* flat, const uint32_t* tok_off, const uint32_t* hit_row,
                                const float* hit_w, size_t total_rows, void* h, const float* gamma, size_t n, size_t rows,
                                float eps, int dtype) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_moe_combine_add_rmsnorm: ctx is NULL");
    CallScope s(c);
    const int es = elem_size(dtype);
    if (!es) return fail(APK_DECLINE_UNSUPPORTED, "apk_moe_combine_add_rmsnorm: dtype %d", dtype);
    if (rows == 0) return APK_OK;
    if (!x || !flat || !hit_row || !hit_w || (h && !gamma))
        return fail(APK_DECLINE_NULL, "apk_moe_combine_add_rmsnorm: NULL tensor");
    // no tok_off list: every token has the same number of hits, total_rows / rows of them, token t's at [t*k, (t+1)*k)
    if (!tok_off && total_rows % rows)
        return fail(APK_DECLINE_SHAPE, "apk_moe_combine_add_rmsnorm: without tok_off every token has total_rows / rows hits, and %zu is "
                                       "not a multiple of %zu", total_rows, rows);
    const size_t vec = 16 / es;
    if (n == 0 || n % vec) return fail(APK_DECLINE_SHAPE, "apk_moe_combine_add_rmsnorm: n=%zu is not a multiple of %zu", n, vec);
    if (!aligned16(x) || !aligned16(flat) || (h && !aligned16(h)) || (gamma && !aligned16(gamma)))
        return fail(APK_DECLINE_SHAPE, "apk_moe_combine_add_rmsnorm: tensors must be 16-byte aligned");
    if (rows > 0x7fffffffu || n > 0x7fffffffu || total_rows > 0xffffffffu)
        return fail(APK_DECLINE_SHAPE, "apk_moe_combine_add_rmsnorm: too large");
    const size_t nchunks = n / vec;
    int nch = 0;
    size_t waves = 0;
    for (int cand : {1, 2, 4}) {
        const size_t w = (nchunks + 64 * (size_t)cand - 1) / (64 * (size_t)cand);
        if (w * 64 > 1024) continue;
        nch = cand;
        waves = w;
        if (rows * w <= 2048) break;
    }
    if (!nch) return fail(APK_DECLINE_SHAPE, "apk_moe_combine_add_rmsnorm: row of %zu elements is too long", n);
    if (int rc = set_device(c)) return rc;
    int n_i = (int)n;
    uint32_t total32 = (uint32_t)total_rows;
    uint32_t uniform_k = tok_off ? 0u : (uint32_t)(total_rows / rows);
    void* args[] = {&x, &flat, &tok_off, &hit_row, &hit_w, &total32, &h, &gamma, &n_i, &eps, &c->fault_dev, &uniform_k};
    const std::string which = std::string("apk_combine_add_rmsnorm_") + (dtype == APK_F32 ? "f32" : "f16") + "_c" + std::to_string(nch);
    return launch(c, which, (unsigned)rows, (unsigned)(waves * 64), 0, args);
}

int apk_argmax_rows(apk_ctx* c, const float* logits, size_t rows, size_t n, uint32_t* out) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_argmax_rows: ctx is NULL");
    CallScope s(c);
    if (rows == 0) return APK_OK;
    // the argument checks come before anything is allocated or declined for the scratch's sake
    if (!logits || !out) return fail(APK_DECLINE_NULL, "apk_argmax_rows: NULL tensor");
    if (n == 0 || n > 0xffffffffu || rows > (1u << 20)) return fail(APK_DECLINE_SHAPE, "apk_argmax_rows: sizes out of range");
    if (int rc = set_device(c)) return rc;
    if (rows > c->argmax_rows_cap) {
        if (c->capturing || c->graphs_with_argmax)
            return fail(APK_DECLINE_CAPTURE, "apk_argmax_rows: the scratch would have to grow %s",
                        c->capturing ? "inside a recording (run once unrecorded first)"
                                     : "while a recorded graph holds its address (destroy the graph first)");
        HIP_TRY(hipStreamSynchronize(c->stream));  // a previous launch may still use the old scratch
        if (c->argmax_scratch) (void)hipFree(c->argmax_scratch);
        c->argmax_scratch = nullptr;
        c->argmax_rows_cap = 0;
        const size_t cap = rows < 256 ? 256 : rows;
        HIP_TRY(hipMalloc(&c->argmax_scratch, cap * 128));
        HIP_TRY(hipMemsetAsync(c->argmax_scratch, 0, cap * 128, c->stream));
        c->argmax_rows_cap = cap;
    }
    if (c->capturing) c->capture_argmax = true;
    return argmax_locked(c, logits, rows, n, out, c->argmax_scratch, false);
}

/* ------------------------------------------------------------- launch plans */

int apk_plan_add_rmsnorm_rows(size_t n, size_t rows, int dtype, apk_plan* plan) {
    if (!plan) return fail(APK_DECLINE_NULL, "apk_plan_add_rmsnorm_rows: plan is NULL");
    return plan_add_rmsnorm(n, rows, dtype, plan);
}

int apk_plan_postnorm_add_rmsnorm_rows(size_t n, size_t rows, int dtype, apk_plan* plan) {
    if (!plan) return fail(APK_DECLINE_NULL, "apk_plan_postnorm_add_rmsnorm_rows: plan is NULL");
    return plan_add_rmsnorm(n, rows, dtype, plan, true);
}

int apk_plan_qknorm_rope(size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, int adjacent_pairs, int dtype,
                         int with_kv_store, apk_plan* plan) {
    if (!plan) return fail(APK_DECLINE_NULL, "apk_plan_qknorm_rope: plan is NULL");
    return plan_qknorm_rope(rows, n_q, n_kv, head_dim, rot_dim, adjacent_pairs ? 1 : 0, dtype, with_kv_store != 0, plan);
}

int apk_plan_attn_prologue_rows(const apk_attn_prologue* a, apk_plan* plan) {
    if (!plan || !a) return fail(APK_DECLINE_NULL, "apk_plan_attn_prologue_rows: NULL argument");
    const bool store = a->k_cache || a->v_cache || a->cache_pos;
    const bool bias = a->q_bias || a->k_bias || (store && a->v_bias);
    return plan_qknorm_rope(a->rows, a->n_q, a->n_kv, a->head_dim, a->rot_dim, a->adjacent_pairs ? 1 : 0, a->dtype, store, plan, bias,
                            a->q_norm || a->k_norm);
}

int apk_plan_scatter_rows(size_t rows, size_t k, size_t cols, int dtype, apk_plan* plan) {
    if (!plan) return fail(APK_DECLINE_NULL, "apk_plan_scatter_rows: plan is NULL");
    return plan_scatter(rows, k, cols, dtype, plan);
}

int apk_plan_embed_rows(int fmt, size_t n_in, size_t t, int out_dtype, apk_plan* plan) {
    if (!plan) return fail(APK_DECLINE_NULL, "apk_plan_embed_rows: plan is NULL");
    return plan_embed(fmt, n_in, t, out_dtype, plan);
}

size_t apk_kernel_count(void) { return all_kernel_names().size(); }

int apk_kernel_name(size_t i, char* name, size_t cap) {
    const std::vector<std::string> v = all_kernel_names();
    if (!name || cap == 0) return fail(APK_DECLINE_NULL, "apk_kernel_name: name is NULL");
    if (i >= v.size()) return fail(APK_DECLINE_RANGE, "apk_kernel_name: %zu of %zu", i, v.size());
    snprintf(name, cap, "%s", v[i].c_str());
    return APK_OK;
}

int apk_copy(apk_ctx* c, const void* src, void* dst, size_t bytes) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_copy: ctx is NULL");
    CallScope s(c);
    if (bytes == 0) return APK_OK;
    if (!src || !dst) return fail(APK_DECLINE_NULL, "apk_copy: NULL tensor");
    if (bytes % 16 || !aligned16(src) || !aligned16(dst)) return fail(APK_DECLINE_SHAPE, "apk_copy: whole 16-byte tiles only");
    if (int rc = set_device(c)) return rc;
    uint64_t nvec = bytes / 16;
    const unsigned block = stream_block(nvec);
    const uint64_t grid = (nvec + block - 1) / block;
    if (grid > 0x7fffffffu) return fail(APK_DECLINE_SHAPE, "apk_copy: too large");
    void* args[] = {&src, &dst, &nvec};
    return launch(c, "apk_copy", (unsigned)grid, block, 0, args);
}

}  // extern "C"
#pragma GCC visibility pop

// (hidden: shared with apk_noalloc.hip, not part of the C ABI)
// The launch both argmax entries share; scratch: 128 bytes per row.
int apk_argmax_launch(apk_ctx* c, const float* logits, size_t rows, size_t n, uint32_t* out, void* scratch, bool clear_first) {
    if (!c) return fail(APK_DECLINE_NULL, "apk_argmax_rows: ctx is NULL");
    CallScope s(c);
    return argmax_locked(c, logits, rows, n, out, scratch, clear_first);
}

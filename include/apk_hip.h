/*
 * libapk_hip.so -- C ABI of the MI355X (gfx950) implementation of allpaka's fused
 * per-layer transformer ops.  This is the boundary an `allpaka_backend::gpu::hip`
 * module (a sibling of gpu/metal, gpu/cuda and gpu/stub, selected in
 * crates/allpaka-backend/src/gpu/mod.rs:13-26) binds through `extern "C"`.
 *
 * Conventions
 *   * Every entry returns an int status and never aborts:
 *       0   APK_OK
 *       >0  declined (apk_decline): the request is outside what the device path
 *           takes; nothing was launched, no caller memory was touched, and the
 *           caller runs its CPU path -- the reference's "decline, never fail"
 *           rule (gpu/stub.rs:37-217, accel.rs:69-102, gpu/types.rs:243-255).
 *       <0  -(hipError_t): the HIP runtime failed.
 *     apk_last_error() returns a thread-local description of the last non-zero
 *     status.
 *   * All tensor pointers are DEVICE pointers unless a name ends in `_host`.
 *     Tensors are dense row-major.  Work is enqueued on the context's single
 *     stream and is asynchronous; apk_sync() waits for it.  Calls on one context
 *     serialise on an internal mutex, like the reference's process-wide backend
 *     (gpu/cuda/runtime/device.rs:267, 944-948).
 *   * dtype selects the ACTIVATION storage type: APK_F32 is the reference's only
 *     activation type; APK_F16 stores activations as IEEE half (widen -> the
 *     same f32/f64 arithmetic -> one round-to-nearest-even).  Norm weights,
 *     RoPE tables, router logits and router weights are always f32.
 *   * The device code object is embedded in the library and loaded with
 *     hipModuleLoadData at apk_init; if that fails apk_init fails -- there is no
 *     CPU fallback inside this library.
 */
#ifndef APK_HIP_H
#define APK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct apk_ctx apk_ctx;

enum apk_dtype { APK_F32 = 0, APK_F16 = 1 };

/* Positive statuses: why a request was declined (cf. DeclineReason, accel.rs:9-67). */
enum apk_decline {
    APK_OK = 0,
    APK_DECLINE_UNSUPPORTED = 1, /* format / dtype / head_dim / n_expert the device path does not take */
    APK_DECLINE_SHAPE = 2,       /* sizes inconsistent or not a whole number of blocks / 16-byte tiles  */
    APK_DECLINE_NULL = 3,        /* a required pointer is NULL                                         */
    APK_DECLINE_RANGE = 4,       /* an index is out of range (host-checked ids)                        */
    APK_DECLINE_NO_DEVICE = 5,   /* no usable GPU / disabled by ALLPAKA_NO_GPU (capability.rs:58-61)   */
    APK_DECLINE_NOT_ATTACHED = 6, /* host address is not inside an attached mapping                   */
    APK_DECLINE_CAPTURE = 7       /* not possible while (or: only while) the stream is being recorded  */
};

/* What an entry would launch for a shape: the kernel of the code object, its grid and workgroup size.
 * Filled by the apk_plan_* functions below, which need neither a context nor a GPU: the entries launch
 * exactly what these return, so the host's choice of launch shape can be checked on any machine. */
typedef struct apk_plan {
    char kernel[64];          /* kernel name in the code object; "" when there is nothing to launch       */
    unsigned grid, block;     /* workgroups, lanes per workgroup                                           */
    unsigned shmem;           /* dynamic LDS bytes                                                         */
    unsigned variant;         /* entry-specific code path (0 when the entry has one)                       */
    unsigned tiles_per_lane;  /* 16-byte tiles (or passes) a lane takes                                    */
    unsigned waves_per_row;   /* waves that share one row (0 where rows are not the unit)                  */
    unsigned rows_per_block;  /* rows (or row items) a workgroup takes when each wave or lane group owns one */
    unsigned lanes_per_row;   /* lanes that cover one row or one head                                      */
    unsigned slices_per_row;  /* workgroup-sized slices a row is cut into (0: workgroups are not tied to rows) */
    unsigned items;           /* work items of the launch before it is rounded up to whole workgroups      */
} apk_plan;

/* Unified dequant format codes -- the exact integers of gpu::common::dq_fmt
 * (crates/allpaka-backend/src/gpu/common.rs:47-61). */
enum apk_dq_fmt {
    APK_FMT_Q4K = 0, APK_FMT_Q5K = 1, APK_FMT_Q6K = 2, APK_FMT_Q8_0 = 3, APK_FMT_Q2K = 4,
    APK_FMT_Q3K = 5, APK_FMT_Q5_0 = 6, APK_FMT_F16 = 7, APK_FMT_F32 = 8, APK_FMT_BF16 = 9
};

/* Bits of the device status word (apk_take_faults). */
enum apk_fault {
    APK_FAULT_TOKEN_RANGE = 1,  /* an embedding id >= vocab was met on the device  */
    APK_FAULT_EXPERT_RANGE = 2, /* a routed expert id >= n_expert                  */
    APK_FAULT_ROW_RANGE = 4,    /* a gather / scatter row index out of range       */
    APK_FAULT_CACHE_RANGE = 8   /* a KV-cache position >= capacity                 */
};

/* ------------------------------------------------------------ life cycle ---- */

/* Creates the backend on `device`: loads the embedded gfx950 code object
 * (hipModuleLoadData), creates the stream.  Replaces the lazy singleton behind
 * gpu::attach / init_error (gpu/stub.rs:37-55, gpu/cuda/mod.rs:41-44).
 * ALLPAKA_NO_GPU set to a non-empty value other than "0" => APK_DECLINE_NO_DEVICE. */
int apk_init(int device, apk_ctx** out);
int apk_shutdown(apk_ctx* ctx);
/* Waits for everything enqueued so far; time spent here is counted as wait_ns. */
int apk_sync(apk_ctx* ctx);
/* The raw hipStream_t the context launches on (for callers that record their own
 * events or order other work against it). */
void* apk_stream(apk_ctx* ctx);
const char* apk_last_error(void);
/* (calls, dispatches, encode_ns, wait_ns) since apk_init -- gpu::stats
 * (gpu/common.rs:24-31). Any pointer may be NULL. */
int apk_stats(apk_ctx* ctx, uint64_t* calls, uint64_t* dispatches, uint64_t* encode_ns, uint64_t* wait_ns);
/* Reads and clears the device status word (synchronises the stream). */
int apk_take_faults(apk_ctx* ctx, uint32_t* faults);

/* Block geometry of a format: bytes of a row of n_in elements, or 0 when the type
 * is unknown or n_in is not a whole number of blocks -- gpu::common::row_bytes
 * (gpu/common.rs:63-68), GgmlType::expected_bytes (allpaka-dtype/src/lib.rs:112-124). */
size_t apk_row_bytes(int fmt, size_t n_in);
/* gpu::can_embed_on_gpu(ty, bytes, n_in) (gpu/stub.rs:85-87): 1 when
 * apk_embed_rows takes this format and row length, else 0. */
int apk_can_embed(int fmt, size_t n_in);

/* -------------------------------------------------------------- memory ------ */

int apk_malloc(apk_ctx* ctx, size_t bytes, void** dev_out);
int apk_free(apk_ctx* ctx, void* dev);
/* Stream-ordered copies; the host buffer must stay valid until apk_sync. */
int apk_h2d(apk_ctx* ctx, void* dev_dst, const void* host_src, size_t bytes);
int apk_d2h(apk_ctx* ctx, void* host_dst, const void* dev_src, size_t bytes);
/* gpu::attach(mapping) / detach (gpu/stub.rs:37-41): copies a host weight mapping to device memory and keys it by
 * host address, so weights are then named by their host address inside the mapping
 * (gpu/cuda/runtime/select.rs:80-84).  The reference's ownership rules (gpu/cuda/runtime/device.rs:588-621): a
 * mapping is keyed by (host_base, len) and counts its owners -- attaching the same key again adds an owner, no
 * copy; a range inside an attached mapping succeeds without a copy and without a count; a range that overlaps one
 * without lying inside it is declined (APK_DECLINE_SHAPE).  apk_detach_range drops one owner of exactly that key
 * (apk_detach: of whatever mapping starts at host_base); the last owner frees the device copy after the stream has
 * drained.  Unknown keys are APK_DECLINE_NOT_ATTACHED.  The reference drops its own recorded graphs on the last
 * detach (they bake in device addresses, and a new file attached at the same host address must never run on the old
 * copy: gpu/cuda/mod.rs:51-54); recorded graphs here belong to the caller, so the last detach of a mapping marks
 * every live apk_graph that was recorded while the mapping was attached as stale: apk_graph_launch declines it
 * (APK_DECLINE_NOT_ATTACHED, nothing launched) until it is destroyed.  Graphs recorded before the mapping was
 * attached cannot hold its addresses and keep working. */
int apk_attach(apk_ctx* ctx, const void* host_base, size_t len);
int apk_detach(apk_ctx* ctx, const void* host_base);
int apk_detach_range(apk_ctx* ctx, const void* host_base, size_t len);
/* Owners of the mapping attached as exactly (host_base, len); 0 when it is not attached (gpu::is_attached, per mapping). */
int apk_attached_owners(apk_ctx* ctx, const void* host_base, size_t len, size_t* owners);
/* Device address of a host address inside an attached mapping (resolve_w, gpu/cuda/runtime/select.rs:80-84);
 * a range that is not wholly inside one is APK_DECLINE_NOT_ATTACHED and *dev_out is NULL. */
int apk_resolve(apk_ctx* ctx, const void* host_ptr, size_t len, void** dev_out);

/* Elapsed device time between two points of the stream (hipEvent based). */
int apk_timer_begin(apk_ctx* ctx);
int apk_timer_end(apk_ctx* ctx, float* ms_out);

/* ------------------------------------------------------ record / replay ---- */

/* Records the ops enqueued between begin and end into a HIP graph instead of
 * running them, and replays the whole chain with ONE submission: the launch-bound
 * decode chain (a few small kernels per layer, tens of layers) pays the host's
 * per-launch cost once.  Replaces the stream capture of the reference's CUDA host
 * (begin_capture in prefill_begin, gpu/cuda/prefill.rs:52-66; `graph.launch()` in
 * prefill_replay, :71-108; drop_pf_graph, gpu/cuda/runtime/device.rs:626-631).
 * As there, a graph bakes in every pointer and size its ops were called with, and
 * nothing may allocate, copy to or from the host, or wait inside a recording:
 * apk_sync, apk_malloc, apk_free, apk_h2d, apk_d2h, apk_attach, apk_detach,
 * apk_take_faults, apk_timer_*, apk_embed_rows_host_ids and an apk_argmax_rows or a
 * large-batch apk_moe_permute that would have to grow its scratch return APK_DECLINE_CAPTURE and record nothing
 * (run the chain once unrecorded first, as the reference does).  A declined op
 * leaves the recording intact.  One recording per context at a time. */
typedef struct apk_graph apk_graph;
int apk_capture_begin(apk_ctx* ctx);
/* Ends the recording and instantiates it; *out is NULL on any non-zero status. */
int apk_capture_end(apk_ctx* ctx, apk_graph** out);
/* Ends the recording and throws it away (prefill_abort, gpu/cuda/prefill.rs:180). */
int apk_capture_abort(apk_ctx* ctx);
/* Enqueues one replay on the context's stream (asynchronous, ordered like an op).  APK_DECLINE_NOT_ATTACHED for a
 * graph recorded while a mapping was attached that has been freed since (see apk_detach_range). */
int apk_graph_launch(apk_ctx* ctx, apk_graph* graph);
/* Number of kernel launches one replay performs. */
int apk_graph_nodes(apk_graph* graph, size_t* nodes);
/* Waits for the stream, then frees the graph. */
int apk_graph_destroy(apk_ctx* ctx, apk_graph* graph);

/* ----------------------------------------------------------------- ops ------ */

/* Embedding gather with the dequant fused in: out[t,:] = dequant(row ids[t]).
 * Replaces QuantMat::row_into over the token loop (quantmat/mod.rs:75-89; callers
 * model/prefill.rs:92-106, model/decode.rs:422-431) and the reference's
 * embed_row_f32_dtoken kernels (token id read on the device).
 * table: [vocab][apk_row_bytes(fmt,n_in)] bytes, 16-byte aligned; ids: u32[t];
 * out: [t][n_in] of out_dtype.  An id >= vocab leaves its row untouched and
 * raises APK_FAULT_TOKEN_RANGE.  All ten formats of apk_dq_fmt are taken, decoded straight from
 * global memory (F16 / BF16 staged through LDS); n_in must be a multiple of 8, and an F16 / BF16
 * row must fit 64 KiB (apk_can_embed tells). */
int apk_embed_rows(apk_ctx* ctx, int fmt, const void* table, size_t vocab, size_t n_in, const uint32_t* ids,
                   size_t t, void* out, int out_dtype);
/* The same followed by `*v *= scale` in f32 when scale != 1 (before the narrowing of an
 * fp16 output): the embedding multiplier of models that scale their token embeddings
 * (model/prefill.rs:107-109, model/decode.rs:427-429; the reference keeps such models on
 * the CPU gather, model/decode.rs:93). */
int apk_embed_rows_scaled(apk_ctx* ctx, int fmt, const void* table, size_t vocab, size_t n_in, const uint32_t* ids,
                          size_t t, float scale, void* out, int out_dtype);
/* Same with the ids on the host: range-checked BEFORE anything is enqueued
 * (APK_DECLINE_RANGE), as the reference's callers reject token >= vocab first.  One id (a decode
 * step whose sampler runs on the host) travels as a kernel argument; more are staged through a
 * pinned buffer of the context, which waits for the previous use of that buffer. */
int apk_embed_rows_host_ids(apk_ctx* ctx, int fmt, const void* table, size_t vocab, size_t n_in,
                            const uint32_t* ids_host, size_t t, void* out, int out_dtype);
/* The rows [row0, row0 + count) of a quantized matrix of n_rows rows, dequantized in place of a
 * gather: out[i, :] = dequant(row row0 + i), no id list.  Replaces QuantMat::row_into over a
 * range (quantmat/mod.rs:75-89, dequant.rs:26-92) and the reference's dequant_rows_f16 kernel,
 * which widens a weight matrix to fp16 ahead of a dense GEMM (gpu/cuda/kernels.rs:2795-2870,
 * launched from gpu/cuda/runtime/gemm.rs:213-260).  Same formats, alignment and bit-exact results
 * as apk_embed_rows; a range outside the matrix is declined (APK_DECLINE_RANGE). */
int apk_dequant_rows(apk_ctx* ctx, int fmt, const void* table, size_t n_rows, size_t n_in, size_t row0, size_t count,
                     void* out, int out_dtype);

/* Residual add on its own: a[i] += b[i].  Replaces ops::add_assign_slice / add_assign_par
 * (ops/blas.rs:105-213) where no norm follows (where one does, apk_add_rmsnorm_rows does
 * both in one pass).  Any n; bit-exact (fp16: widen, add in f32, one rounding). */
int apk_add_assign(apk_ctx* ctx, void* a, const void* b, size_t n, int dtype);

/* Scaled accumulate on its own: dst[i] = fma(src[i], scale, dst[i]), one rounding.  Replaces ops::add_scaled_slice
 * (ops/blas.rs:25-102), the step the decode MoE combine repeats per picked expert, best first, and once more with
 * scale 1 for the shared expert (model/moe.rs:500-509); a whole batch's combine is apk_moe_combine_add_rmsnorm.
 * dst, src: n elements of dtype, two tensors; fp16 rows take the f32 fma rounded once. */
int apk_add_scaled(apk_ctx* ctx, void* dst, const void* src, size_t n, float scale, int dtype);
/* Softmax over rows of f32 in place.  Replaces ops::softmax (ops/activation.rs:5-16) per
 * row; the router's softmax is fused into apk_route_topk, this is the op on its own.
 * Rows of at most 4096 (router widths): the reference adds the exponentials one after the
 * other in f32, which a parallel sum matches to 1e-5 only for short rows; longer declined. */
int apk_softmax_rows(apk_ctx* ctx, float* x, size_t rows, size_t n);

/* Residual add + RMSNorm over rows: x += delta (skipped when delta is NULL), then
 * h = rmsnorm(x) * gamma.  Replaces ops::add_assign_slice followed by
 * ops::rmsnorm_into / rmsnorm_rows_into (ops/blas.rs:105-178, ops/norm.rs:193-304;
 * call sites model/decode.rs:584,764, model/prefill.rs:155,308-314).
 * x, delta, h: [rows][n] of dtype (h may alias x when delta is NULL);
 * gamma: f32[n].  Rows of any length are taken: whole 16-byte tiles up to 20 480 elements by
 * the tiled kernels, anything else by an element-wise two-pass kernel. */
int apk_add_rmsnorm_rows(apk_ctx* ctx, void* x, const void* delta, void* h, const float* gamma, size_t n,
                         size_t rows, float eps, int dtype);

/* The sandwich norm of the Gemma family, then the next norm, in one pass:
 *   x[r] += rmsnorm(delta[r]) * post_gamma;   h[r] = rmsnorm(x[r]) * gamma.
 * Replaces ops::rmsnorm(projected, post_norm, eps); ops::add_assign_slice(x, projected) and the
 * ops::rmsnorm_into that follows (model/decode.rs:581-584 and :771-775 with :762-764; the reference's CUDA
 * rmsnorm_add_f32, gpu/cuda/kernels.rs:376-406; GroupedCombine.post_norm, gpu/types.rs:437-440).  Same
 * arithmetic as apk_add_rmsnorm_rows for both norms; with fp16 activations the normalised delta is
 * rounded to fp16 before the add, as the reference's in-place row would be.  One launch where
 * apk_add_rmsnorm_rows would take its tiled kernels (the delta is then left unchanged); other rows run
 * the reference's two steps and overwrite delta with its normalised form.  x, delta, h distinct. */
int apk_postnorm_add_rmsnorm_rows(apk_ctx* ctx, void* x, void* delta, const float* post_gamma, void* h, const float* gamma,
                                  size_t n, size_t rows, float eps, int dtype);

/* Per-head QK-norm then NeoX RoPE, in place.  Replaces the loop
 * ops::rmsnorm(head, w, eps); ops::rope_neox_cached_from_array(head, rope_row)
 * over every q and k head of every row (model/attention.rs:131-165,
 * ops/norm.rs:115-187, ops/rope.rs:70-81).
 * q: [rows][n_q*head_dim], k: [rows][n_kv*head_dim] of dtype; qw, kw: f32[head_dim]
 * or NULL (no norm for that tensor); rope: f32 [rows][rot_dim/2][2] = [sin, cos]
 * per row (the session table rows, model/session.rs:34-50).
 * rot_dim (even, <= head_dim) is the rotary width: pairs (i, i + rot_dim/2) rotate and
 * channels >= rot_dim are normalised and pass through (partial rotary, rope.rs:66-81).
 * head_dim in {64,128,256} with a rotary width of whole 16-byte tiles (rot_dim/2 a multiple of
 * 8 fp16 / 4 f32 elements; rot_dim itself for adjacent pairs) takes the tiled kernels; rot_dim = 0
 * and any other geometry take an element-wise kernel (a wave per head, 2.5-4x slower). */
int apk_qknorm_rope_neox(apk_ctx* ctx, void* q, void* k, const float* qw, const float* kw, const float* rope,
                         size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, float eps,
                         int dtype);
/* The same with the adjacent-pair rotation (2i, 2i+1) of RopeStyle::Norm models:
 * ops::rope_norm_cached_from_array (ops/rope.rs:52-64), selected per model in
 * rope_from_arrays (model/attention.rs:62-67).  The same kernel choice: tiled for a whole head of
 * 64 / 128 / 256, element-wise otherwise. */
int apk_qknorm_rope_norm(apk_ctx* ctx, void* q, void* k, const float* qw, const float* kw, const float* rope,
                         size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, float eps,
                         int dtype);

/* apk_qknorm_rope_neox with the K/V cache store fused in: after the rotation, row r's k
 * (all n_kv heads) and the same row of v are narrowed to fp16 (RNE) into cache row
 * cache_pos[r].  Replaces the QK-norm+RoPE loop followed by KvCache::store_at(layer,
 * base_pos + i, k_row, v_row) (crates/allpaka-model/src/kv.rs:682-697; call site
 * model/attention.rs:170-200); every accelerator path of the reference fuses the same
 * store (rmsnorm_rope_qk_store_table_dpos, gpu/cuda/kernels.rs:687-765; qk_prep,
 * gpu/shaders/kernels.metal:7705-7712).  q and k are still updated in place.
 * v: [rows][n_kv*head_dim] of dtype (read only); cache_pos: u32[rows] on the device;
 * k_cache, v_cache: fp16 [capacity][n_kv*head_dim] (one layer's K and V planes).
 * A position >= capacity skips that row's cache store and raises APK_FAULT_CACHE_RANGE
 * (the reference asserts "position past capacity").  NeoX over a whole head of
 * 64/128/256 only; other geometries are declined (run the two steps separately). */
int apk_qknorm_rope_kv_store(apk_ctx* ctx, void* q, void* k, const void* v, const float* qw, const float* kw,
                             const float* rope, const uint32_t* cache_pos, void* k_cache, void* v_cache,
                             size_t capacity, size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim,
                             float eps, int dtype);

/* The same with adjacent rotary pairs (RopeStyle::Norm, as apk_qknorm_rope_norm): the chunk prologue of
 * the Llama-family layouts with the cache store fused in. */
int apk_qknorm_rope_norm_kv_store(apk_ctx* ctx, void* q, void* k, const void* v, const float* qw, const float* kw,
                                  const float* rope, const uint32_t* cache_pos, void* k_cache, void* v_cache,
                                  size_t capacity, size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim,
                                  float eps, int dtype);

/* The same step with the rotary angles taken from the rows' positions INSIDE the launch, for a decode-sized batch
 * (rows <= 64): [sin, cos] of pair i of row r is sincos((positions[r] as f32) * inv_freq[i]) (ops::rope_sin_cos,
 * ops/rope.rs:18-22), the values apk_rope_table writes, so the call equals apk_rope_table(positions, inv_freq, ...)
 * followed by apk_qknorm_rope_neox / _norm (adjacent_pairs != 0) on that table -- without the table and without its
 * launch.  Replaces the reference's device-angle kernels rmsnorm_rope_freq_dpos / rmsnorm_rope_store_freq_dpos
 * (gpu/cuda/kernels.rs:577-671; set_rope_inv_freq / has_device_rope_freq, gpu/stub.rs), which read the position and
 * inv_freq in the kernel so that one recorded graph serves every token.  positions: u32[rows] and inv_freq:
 * f32[rot_dim/2], both on the device.  With k_cache and v_cache (both or neither; then v is required) the rotated k
 * rows and the rows of v are also narrowed to fp16 into cache row positions[r], as apk_qknorm_rope_kv_store does with
 * cache_pos = positions; a position >= capacity skips that row's store and raises APK_FAULT_CACHE_RANGE.  Any head
 * geometry, partial rotary included.  More than 64 rows: APK_DECLINE_SHAPE (build the table once per step with
 * apk_rope_table and run the table form, which is the faster one from there on).  May be recorded. */
int apk_qknorm_rope_pos(apk_ctx* ctx, void* q, void* k, const void* v, const float* qw, const float* kw,
                        const uint32_t* positions, const float* inv_freq, void* k_cache, void* v_cache, size_t capacity,
                        size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, int adjacent_pairs,
                        float eps, int dtype);

/* Layer prologue as ONE launch: apk_add_rmsnorm_rows(x, delta, h, gamma, n, rows) and
 * apk_qknorm_rope_neox(q, k, qw, kw, rope, rows, ...) with the same arguments and the
 * same results, as two independent jobs in one grid (the reference's accelerators fuse
 * the same pair of ops into their per-token command buffer, e.g. residual_norm + qk_prep,
 * crates/allpaka-backend/src/gpu/metal/decode.rs:670; here q/k are inputs, a QKV
 * projection sits between the two in a real layer).  Single launch when a row is at most
 * 1024 16-byte tiles and rows * ceil(tiles/64) <= 2048 (decode and batched-decode
 * shapes); otherwise it runs the two launches itself. */
int apk_layer_prologue(apk_ctx* ctx, void* x, const void* delta, void* h, const float* gamma, size_t n, void* q,
                       void* k, const float* qw, const float* kw, const float* rope, size_t rows, size_t n_q,
                       size_t n_kv, size_t head_dim, size_t rot_dim, float eps, int dtype);

/* inv_freq[i] = base.powf(-2 i / rot_dim) for i < rot_dim / 2, in f32 on the host: ops::rope_inv_freq
 * (ops/rope.rs:8-12), which the reference computes once at load with the platform's powf -- the
 * same libm symbol this uses.  No context, no GPU. */
int apk_rope_inv_freq(size_t rot_dim, float base, float* inv_freq);

/* Builds RoPE table rows on the device: table[r][i] = [sin, cos](pos[r] as f32 *
 * inv_freq[i]).  Replaces ops::rope_sin_cos per position (ops/rope.rs:18-22;
 * Session::ensure_rope_cache, model/session.rs:34-50; gpu::multi_stage's staging
 * of positions, gpu/stub.rs:181-183).  positions: u32[rows]; inv_freq: f32[half]. */
int apk_rope_table(apk_ctx* ctx, const uint32_t* positions, const float* inv_freq, size_t rows, size_t half,
                   float* table);

/* SwiGLU in place: gate[i] = silu(gate[i]) * up[i].  Replaces ops::swiglu
 * (ops/activation.rs:57-120, non-aarch64 arm). */
int apk_swiglu(apk_ctx* ctx, void* gate, const void* up, size_t n, int dtype);
/* gate[i] = gelu_tanh(gate[i]) * up[i] in place: GeGLU with the tanh GELU, the FFN gate of the Gemma
 * family.  Replaces ops::geglu_tanh (ops/activation.rs:44-51; chosen instead of swiglu where
 * GroupedCombine.gelu is set, model/moe.rs:122-127, gpu/types.rs:440-443; the reference's CUDA kernel of
 * the same name, gpu/cuda/kernels.rs:361).  Computed as gate * sigmoid(2z) * up, which is the same
 * function without the cancellation of 1 + tanh z: f32 results agree with the reference's to 1e-5
 * relative where 1 + tanh z >= 0.1 and to the reference's own tolerance idiom |a-b| < 1e-5 (1 + |b|)
 * everywhere (for very negative gates its f32 result carries the rounding of its tanh); fp16: 2 ulp
 * where 1 + tanh z >= 0.1, the same idiom on the values elsewhere. */
int apk_geglu_tanh(apk_ctx* ctx, void* gate, const void* up, size_t n, int dtype);

/* MoE router: softmax (sigmoid == 1: sigmoid; sigmoid == 2: the rows hold the scores already) over n_expert
 * logits, top-k by descending selection score (+ bias when given), ties -> lower expert id,
 * weights renormalised over the winners when norm != 0, then * scale.  Replaces
 * model::route_gated / route_gated_into_slice per token (model/moe.rs:524-616,
 * token loop :204-227); with sigmoid == 2, norm != 0, scale 1 and no bias it is the older
 * model::route(probs, k) on softmaxed rows (model/moe.rs:623-658), bit for bit.  logits: f32[rows][n_expert];
 * ids: u32[rows][k]; w: f32[rows][k], both best-first.  n_expert <= 1024, 1 <= k <= min(n_expert, 64). */
int apk_route_topk(apk_ctx* ctx, const float* logits, const float* bias, size_t rows, size_t n_expert, size_t k,
                   int norm, float scale, int sigmoid, uint32_t* ids, float* w);

/* Token -> expert grouping in the CPU order.  Replaces the groups/used/table/tok
 * construction and the CSR inversion of Ffn::moe_batch (model/moe.rs:229-271,
 * :298-309; model/prefill.rs:624-675).  ids, w: [rows][k] from apk_route_topk.
 * table: u32[n_expert][3] = (expert, row0, rows) for the NON-EMPTY experts in
 * ascending order, *n_used of them (a device u32); tok: u32[rows*k] token of each
 * flat row (expert-major, token-ascending inside an expert); tok_off: u32[rows+1];
 * hit_row: u32[rows*k], hit_w: f32[rows*k] per-token hit lists in ascending
 * expert order.  n_expert <= 1024, rows*k < 2^31. */
int apk_moe_permute(apk_ctx* ctx, const uint32_t* ids, const float* w, size_t rows, size_t k, size_t n_expert,
                    uint32_t* table, uint32_t* n_used, uint32_t* tok, uint32_t* tok_off, uint32_t* hit_row,
                    float* hit_w);

/* apk_route_topk followed by apk_moe_permute, with the same arguments and the same results bit for
 * bit; ONE launch for a decode-sized batch (rows <= 16), where the two launches
 * cost a launch latency each and the second waits for the first.  The reference's accelerators route
 * and group inside one command buffer as well (GroupedRoute of a GroupedFfnReq, gpu/types.rs:406-416,
 * :446-467; the Metal route_scatter / route_fused kernels, gpu/shaders/kernels.metal:2223-2424).  Larger
 * batches run the two entries: a single launch whose last-arriving workgroup groups the picks was measured
 * at 1024 tokens x 128 experts and is slower (three dependent device-scope round trips -- write-through
 * acknowledgement, arrival count, re-read of the picks -- cost more than the second launch they replace). */
int apk_route_group(apk_ctx* ctx, const float* logits, const float* bias, size_t rows, size_t n_expert, size_t k,
                    int norm, float scale, int sigmoid, uint32_t* ids, float* w, uint32_t* table, uint32_t* n_used,
                    uint32_t* tok, uint32_t* tok_off, uint32_t* hit_row, float* hit_w);

/* The shared expert of GLM-style MoE layers in the per-token hit lists: every token gets one more hit, after
 * its routed ones, of weight 1.0 at flat row total_rows + token (the shared FFN's rows sit right after the
 * experts' rows).  Replaces model/prefill.rs:621-635 (h.push((total_rows + i, 1.0))) and the flattening
 * :658-675.  tok_off: u32[rows+1], hit_row / hit_w: [tok_off[rows]] as apk_moe_permute writes them (any CSR
 * will do); the outputs hold tok_off[rows] + rows hits and must be arrays of their own.  apk_moe_combine_add_rmsnorm
 * then takes the lengthened lists with total_rows + rows flat rows; apk_gather_rows / apk_scatter_rows keep
 * the routed lists. */
int apk_moe_shared_hits(apk_ctx* ctx, const uint32_t* tok_off, const uint32_t* hit_row, const float* hit_w, size_t rows,
                        size_t total_rows, uint32_t* tok_off_out, uint32_t* hit_row_out, float* hit_w_out);

/* dst[r,:] = src[tok[r],:] -- the gathered expert activations (model/moe.rs:348-352).
 * src: [src_rows][cols], dst: [total_rows][cols] of dtype; cols*sizeof(dtype) must
 * be a multiple of 16. */
int apk_gather_rows(apk_ctx* ctx, const void* src, const uint32_t* tok, size_t src_rows, size_t total_rows,
                    size_t cols, void* dst, int dtype);

/* The same expert-grouped rows produced from the token side with the CSR lists of
 * apk_moe_permute: dst[hit_row[t*k + j], :] = src[t, :] for j < k.  Equal to
 * apk_gather_rows(src, tok, ...) when (tok, hit_row) come from one apk_moe_permute call
 * (model/moe.rs:298-309 builds hit_row as the inverse of tok), and the faster form:
 * each source row is read once.  A hit >= total_rows is skipped and raises
 * APK_FAULT_ROW_RANGE. */
int apk_scatter_rows(apk_ctx* ctx, const void* src, const uint32_t* hit_row, size_t rows, size_t k, size_t total_rows,
                     size_t cols, void* dst, int dtype);

/* MoE combine + residual add + the next RMSNorm in one pass per token row:
 *   out = 0; for each hit j in [tok_off[t], tok_off[t+1]): out = fma(flat[hit_row[j]], hit_w[j], out);
 *   x[t] += out;  h[t] = rmsnorm(x[t]) * gamma.
 * Replaces the per-token ops::add_scaled_slice loop of Ffn::moe_batch (model/moe.rs:298-333;
 * ops/blas.rs:25-102, one fused multiply-add per hit), the residual ops::add_assign_slice
 * (model/decode.rs:775, model/prefill.rs:308) and the next ops::rmsnorm_rows_into
 * (model/prefill.rs:155/314); the reference's accelerators fuse the same three
 * (combine_rows_resnorm, gpu/shaders/kernels.metal:1905-1974; GroupedCombine.next_norm,
 * gpu/types.rs:429-443).  flat: [total_rows][n] expert down-projection rows of dtype;
 * tok_off/hit_row/hit_w: the CSR lists of apk_moe_permute.  tok_off may be NULL when every token has the same
 * number of hits (a routed layer without a shared expert: tok_off[t] would read t * k): the hits of token t are
 * then [t * k, (t + 1) * k) with k = total_rows / rows (total_rows not a multiple of rows: APK_DECLINE_SHAPE), and
 * the launch is faster for the dependent load it no longer makes.  h (and gamma) may be NULL:
 * combine and residual only.  A hit >= total_rows is skipped and raises APK_FAULT_ROW_RANGE. */
int apk_moe_combine_add_rmsnorm(apk_ctx* ctx, void* x, const void* flat, const uint32_t* tok_off,
                                const uint32_t* hit_row, const float* hit_w, size_t total_rows, void* h,
                                const float* gamma, size_t n, size_t rows, float eps, int dtype);

/* Greedy next token per row of logits: the LAST maximum under f32::total_cmp, exactly
 * (0..n).max_by(|a, b| logits[a].total_cmp(&logits[b])) of Model::forward_greedy
 * (model/decode.rs:628-630; ties -> higher index, as the reference's Metal argmax,
 * gpu/shaders/kernels.metal:3726-3728).  logits: f32[rows][n]; out: u32[rows].
 * Uses a small per-context scratch (128 bytes per row, allocated on first use). */
int apk_argmax_rows(apk_ctx* ctx, const float* logits, size_t rows, size_t n, uint32_t* out);

/* apk_argmax_rows for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  No counterpart in the reference (its hosts allocate their arenas up front).  Same result
 * as apk_argmax_rows; allocates nothing, ever: the 128 bytes of scratch per row live in a static device array
 * of the library, 2048 rows = 256 KiB per GPU, held until the process ends.  More than 2048 rows are declined
 * (APK_DECLINE_SHAPE).  May be recorded (apk_capture_begin .. _end).  Every call on a GPU shares that GPU's array:
 * calls that overlap on one GPU -- two contexts, or one context from two host threads without its lock -- race. */
int apk_argmax_rows_noalloc(apk_ctx* ctx, const float* logits, size_t rows, size_t n, uint32_t* out);

/* dst = src, `bytes` a multiple of 16: the plain stream kernel the bandwidth
 * figures of the other kernels are calibrated against. */
int apk_copy(apk_ctx* ctx, const void* src, void* dst, size_t bytes);

/* dst[i] = src[i] converted between the reference's f32 activations and the fp16 storage form: APK_F32 ->
 * APK_F16 is allpaka_dtype::f32_to_f16 (crates/allpaka-dtype/src/lib.rs:151-184: round to nearest even,
 * overflow to infinity, subnormals kept, NaN -> sign | 0x7e00), APK_F16 -> APK_F32 is f16_to_f32 (:129-146:
 * exact, NaN payloads kept); bit for bit, for every input.  The reference's CUDA cast_f32_to_f16 /
 * cast_f16_to_f32 (gpu/cuda/kernels.rs:448, :3625).  Any n; src and dst distinct, 16-byte aligned. */
int apk_cast(apk_ctx* ctx, const void* src, int src_dtype, void* dst, int dst_dtype, size_t n);

/* x[r][i] += bias[i] over rows of length n (add_bias_rows, crates/allpaka-model/src/model/loader.rs:519-523:
 * ops::add_assign_slice(row, bias) per row).  x: [rows][n] of dtype, in place; bias: f32[n]. */
int apk_add_bias_rows(apk_ctx* ctx, void* x, const float* bias, size_t rows, size_t n, int dtype);

/* Everything the reference does to a batch's projected q, k, v rows between the QKV projection and
 * attention, as one call (model/attention.rs:125-165 and the cache store kv.rs:682-697):
 *   add_bias_rows(q, q_bias); add_bias_rows(k, k_bias); add_bias_rows(v, v_bias)      (:125-129; each optional)
 *   per head: ops::rmsnorm(head, q_norm | k_norm, eps) (optional), then the row's rotation  (:131-165)
 *   KvCache::store_at: k and v narrowed to f16 at cache row cache_pos[row]             (optional)
 * Fields as in apk_qknorm_rope_neox / _norm (adjacent_pairs != 0) / _kv_store; the biases are f32
 * [n_q*head_dim] / [n_kv*head_dim], 16-byte aligned, NULL for none.  The cache store is asked for by a
 * non-NULL k_cache (then v, cache_pos, v_cache and capacity are required).  One launch for heads of
 * 64/128/256 with a rotary width of whole tiles; v_bias without the cache store is one more launch
 * (v is not otherwise read), and other head geometries take the element-wise kernel (no cache store there).
 * With biases, fp16 rows are widened, biased, normalised and rotated in f32 and rounded once. */
typedef struct apk_attn_prologue {
    void* q;                 /* [rows][n_q*head_dim] of dtype, in place */
    void* k;                 /* [rows][n_kv*head_dim] of dtype, in place */
    void* v;                 /* [rows][n_kv*head_dim] of dtype: read for the cache store, written only with v_bias; else NULL */
    const float* q_bias;
    const float* k_bias;
    const float* v_bias;
    const float* q_norm;     /* f32[head_dim] or NULL */
    const float* k_norm;
    const float* rope;       /* f32 [rows][rot_dim/2][2] = [sin, cos] */
    const uint32_t* cache_pos; /* [rows] cache row per batch row, or NULL */
    void* k_cache;           /* f16 [capacity][n_kv*head_dim], or NULL: no store */
    void* v_cache;
    size_t capacity;
    size_t rows, n_q, n_kv, head_dim, rot_dim;
    float eps;
    int dtype;
    int adjacent_pairs;      /* 0: NeoX pairs (i, i + rot_dim/2); else pairs (2i, 2i+1) */
} apk_attn_prologue;
int apk_attn_prologue_rows(apk_ctx* ctx, const apk_attn_prologue* args);

/* Launch plans (no context, no GPU; see apk_plan): what apk_add_rmsnorm_rows, apk_postnorm_add_rmsnorm_rows, apk_qknorm_rope_neox /
 * _norm (adjacent_pairs != 0) / _kv_store (with_kv_store != 0), apk_scatter_rows and apk_embed_rows /
 * apk_dequant_rows launch for these sizes.  Return APK_OK with plan filled (kernel "" and grid 0 when
 * the call would be a no-op), or the decline the entry itself would return for the sizes.  (apk_plan_attn_prologue_rows:
 * the launch over q and k; a v_bias without the cache store is one more launch, of the plain bias kernel.)  They have no
 * counterpart in the reference: its hosts size their dispatches inline (e.g. gpu/cuda/runtime/gemm.rs:218-233). */
int apk_plan_add_rmsnorm_rows(size_t n, size_t rows, int dtype, apk_plan* plan);
int apk_plan_postnorm_add_rmsnorm_rows(size_t n, size_t rows, int dtype, apk_plan* plan);
int apk_plan_qknorm_rope(size_t rows, size_t n_q, size_t n_kv, size_t head_dim, size_t rot_dim, int adjacent_pairs, int dtype,
                         int with_kv_store, apk_plan* plan);
int apk_plan_attn_prologue_rows(const apk_attn_prologue* args, apk_plan* plan);
int apk_plan_scatter_rows(size_t rows, size_t k, size_t cols, int dtype, apk_plan* plan);
int apk_plan_embed_rows(int fmt, size_t n_in, size_t t, int out_dtype, apk_plan* plan);
/* The kernels apk_init resolves from the embedded code object: their number, and the i-th name copied into
 * name[cap] (every plan names one of them). */
size_t apk_kernel_count(void);
int apk_kernel_name(size_t i, char* name, size_t cap);

#ifdef __cplusplus
}
#endif
#endif /* APK_HIP_H */

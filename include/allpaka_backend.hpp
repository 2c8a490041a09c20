// Host-side mirror of the reference's operator surface over the C ABI (apk_hip.h).
//
// Same names, argument meaning and error behaviour as `allpaka_backend::ops::*`
// (crates/allpaka-backend/src/ops/{norm,rope,activation,blas}.rs), `QuantMat::{new,row,
// row_into}` (crates/allpaka-backend/src/quantmat/mod.rs:39-89) and `model::route_gated`
// (crates/allpaka-model/src/model/moe.rs:601-616), on HOST slices as the reference's CPU
// callers hold them: each call copies its operands to the device, runs the kernel and
// copies the result back.  That makes these functions drop-in for a call site, not fast
// -- a resident pipeline calls the C ABI with device pointers instead.
//
//   * where the reference panics (length asserts), these throw `Panic`;
//   * where it returns Err (QuantMat, dequant), these throw `Error`;
//   * where an accelerator entry declines (`None`), these throw `Declined{reason}`.
//
// There is no CPU fallback here: without a usable GPU `Gpu::get()` throws Declined.
#pragma once
#include <array>
#include <cstdint>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "apk_hip.h"

namespace allpaka_backend {

struct Panic : std::logic_error { using std::logic_error::logic_error; };      // the reference's assert!/panic!
struct Error : std::runtime_error { using std::runtime_error::runtime_error; }; // the reference's Err(..)
struct Declined : std::runtime_error {                                          // the reference's None / Declined
    int reason;
    Declined(int r, const std::string& m) : std::runtime_error(m), reason(r) {}
};

enum class GgmlType : int { Q4K = 0, Q5K, Q6K, Q8_0, Q2K, Q3K, Q5_0, F16, F32, BF16 };  // = gpu::common::dq_fmt codes
enum class Gating : int { Softmax = 0, Sigmoid = 1 };

inline void check(int rc) {
    if (rc == 0) return;
    if (rc > 0) throw Declined(rc, apk_last_error());
    throw std::runtime_error(std::string("HIP: ") + apk_last_error());
}

// The process-wide backend (the reference's `static GPU: OnceLock<..>`, gpu/cuda/runtime/device.rs:267).
class Gpu {
  public:
    static Gpu& get() {
        static Gpu g;
        return g;
    }
    apk_ctx* ctx() const { return ctx_; }
    Gpu(const Gpu&) = delete;

  private:
    Gpu() { check(apk_init(0, &ctx_)); }
    ~Gpu() { apk_shutdown(ctx_); }
    apk_ctx* ctx_ = nullptr;
};

// A device copy of a host slice for the duration of one call.
template <typename T> class Dev {
  public:
    Dev(const T* host, size_t n) : n_(n) {
        check(apk_malloc(Gpu::get().ctx(), n * sizeof(T), &p_));
        if (host && n) check(apk_h2d(Gpu::get().ctx(), p_, host, n * sizeof(T)));
    }
    explicit Dev(size_t n) : Dev(nullptr, n) {}
    ~Dev() { apk_free(Gpu::get().ctx(), p_); }
    Dev(const Dev&) = delete;
    T* ptr() const { return static_cast<T*>(p_); }
    void read_back(T* host) const {
        check(apk_d2h(Gpu::get().ctx(), host, p_, n_ * sizeof(T)));
        check(apk_sync(Gpu::get().ctx()));
    }

  private:
    void* p_ = nullptr;
    size_t n_;
};

// The accelerator surface's ownership calls (gpu/stub.rs:37-41; gpu/cuda/mod.rs:41-63): a host weight mapping is
// copied to device memory once and weights are then named by their host address inside it.
namespace gpu {
// gpu::attach(mapping) -> bool: false where the reference returns false (no device, or the range overlaps another).
inline bool attach(const uint8_t* mapping, size_t len) { return apk_attach(Gpu::get().ctx(), mapping, len) == APK_OK; }
// gpu::detach(mapping): releases one attach of exactly this mapping; silent when it was not attached, as the reference
// (false then).  Any other status is an error of the device and is thrown: the caller must never believe a mapping
// gone that is still resident.  The last owner frees the copy, and graphs recorded while it was attached decline
// their replays from then on.
inline bool detach(const uint8_t* mapping, size_t len) {
    const int rc = apk_detach_range(Gpu::get().ctx(), mapping, len);
    if (rc == APK_DECLINE_NOT_ATTACHED) return false;
    check(rc);
    return true;
}
// owners of exactly this mapping (0: not attached)
inline size_t owners(const uint8_t* mapping, size_t len) {
    size_t n = 0;
    check(apk_attached_owners(Gpu::get().ctx(), mapping, len, &n));
    return n;
}
// resolve_w (gpu/cuda/runtime/select.rs:80-84): the device address of a host slice inside an attached mapping, or
// nullptr for foreign memory.
inline const void* resolve(const void* host, size_t len) {
    void* dev = nullptr;
    return apk_resolve(Gpu::get().ctx(), host, len, &dev) == APK_OK ? dev : nullptr;
}
}  // namespace gpu

namespace ops {

// ops::rmsnorm(x, weight, eps): in place over one row (norm.rs:115).
inline void rmsnorm(std::vector<float>& x, const std::vector<float>& weight, float eps) {
    if (x.size() != weight.size()) throw Panic("assertion failed: x.len() == weight.len()");
    Dev<float> dx(x.data(), x.size()), dw(weight.data(), weight.size());
    check(apk_add_rmsnorm_rows(Gpu::get().ctx(), dx.ptr(), nullptr, dx.ptr(), dw.ptr(), x.size(), 1, eps, APK_F32));
    dx.read_back(x.data());
}

// ops::rmsnorm_into(dst, src, weight, eps) (norm.rs:193).
inline void rmsnorm_into(std::vector<float>& dst, const std::vector<float>& src, const std::vector<float>& weight, float eps) {
    if (src.size() != weight.size()) throw Panic("assertion failed: src.len() == weight.len()");
    if (dst.size() != src.size()) throw Panic("assertion failed: dst.len() == src.len()");
    Dev<float> ds(src.data(), src.size()), dd(dst.size()), dw(weight.data(), weight.size());
    check(apk_add_rmsnorm_rows(Gpu::get().ctx(), ds.ptr(), nullptr, dd.ptr(), dw.ptr(), src.size(), 1, eps, APK_F32));
    dd.read_back(dst.data());
}

// ops::rmsnorm_rows_into(dst, src, weight, eps): rows = src.len() / weight.len() (norm.rs:275).
inline void rmsnorm_rows_into(std::vector<float>& dst, const std::vector<float>& src, const std::vector<float>& weight, float eps) {
    const size_t n = weight.size(), rows = src.size() / n;
    if (dst.size() < rows * n) throw Panic("dst holds fewer rows than src");
    Dev<float> ds(src.data(), rows * n), dd(rows * n), dw(weight.data(), n);
    check(apk_add_rmsnorm_rows(Gpu::get().ctx(), ds.ptr(), nullptr, dd.ptr(), dw.ptr(), n, rows, eps, APK_F32));
    std::vector<float> out(rows * n);
    dd.read_back(out.data());
    std::copy(out.begin(), out.end(), dst.begin());
}

// ops::add_assign_slice(a, b) immediately followed by ops::rmsnorm_into(h, a, weight, eps): the pair the
// decode loop runs (decode.rs:584 then :764) as one launch.  On the device the residual add only exists in
// this fused form.
inline void add_assign_then_rmsnorm_into(std::vector<float>& a, const std::vector<float>& b, std::vector<float>& h,
                                         const std::vector<float>& weight, float eps) {
    if (a.size() != b.size()) throw Panic("assertion failed: a.len() == b.len()");
    const size_t n = weight.size(), rows = a.size() / n;
    if (h.size() < rows * n) throw Panic("dst holds fewer rows than src");
    Dev<float> da(a.data(), a.size()), db(b.data(), b.size()), dh(rows * n), dw(weight.data(), n);
    check(apk_add_rmsnorm_rows(Gpu::get().ctx(), da.ptr(), db.ptr(), dh.ptr(), dw.ptr(), n, rows, eps, APK_F32));
    da.read_back(a.data());
    std::vector<float> out(rows * n);
    dh.read_back(out.data());
    std::copy(out.begin(), out.end(), h.begin());
}

// The sandwich norm of the Gemma family and the norm that follows it (decode.rs:581-584 / :771-775, then :762-764):
// ops::rmsnorm(delta, post_weight, eps); ops::add_assign_slice(a, delta); ops::rmsnorm_into(h, a, weight, eps) as one
// launch.  `delta` itself is left as it was (the reference normalises it in place; nothing reads it afterwards).
inline void postnorm_add_assign_then_rmsnorm_into(std::vector<float>& a, const std::vector<float>& delta,
                                                  const std::vector<float>& post_weight, std::vector<float>& h,
                                                  const std::vector<float>& weight, float eps) {
    if (a.size() != delta.size()) throw Panic("assertion failed: a.len() == b.len()");
    if (post_weight.size() != weight.size()) throw Panic("assertion failed: x.len() == weight.len()");
    const size_t n = weight.size(), rows = a.size() / n;
    if (h.size() < rows * n) throw Panic("dst holds fewer rows than src");
    Dev<float> da(a.data(), a.size()), dd(delta.data(), delta.size()), dh(rows * n), dw(weight.data(), n), dp(post_weight.data(), n);
    check(apk_postnorm_add_rmsnorm_rows(Gpu::get().ctx(), da.ptr(), dd.ptr(), dp.ptr(), dh.ptr(), dw.ptr(), n, rows, eps, APK_F32));
    da.read_back(a.data());
    std::vector<float> out(rows * n);
    dh.read_back(out.data());
    std::copy(out.begin(), out.end(), h.begin());
}

// ops::rope_inv_freq(head_dim, base) (rope.rs:8-12): host-side, as in the reference.
inline std::vector<float> rope_inv_freq(size_t head_dim, float base) {
    std::vector<float> inv(head_dim / 2);
    check(apk_rope_inv_freq(head_dim, base, inv.data()));
    return inv;
}
// ops::rope_sin_cos (rope.rs:18-22) per position; the table rows for a batch of positions are built on the device:
inline std::vector<std::array<float, 2>> rope_sin_cos_rows(const std::vector<uint32_t>& positions, const std::vector<float>& inv_freq) {
    Dev<uint32_t> dp(positions.data(), positions.size());
    Dev<float> di(inv_freq.data(), inv_freq.size()), dt(positions.size() * inv_freq.size() * 2);
    check(apk_rope_table(Gpu::get().ctx(), dp.ptr(), di.ptr(), positions.size(), inv_freq.size(), dt.ptr()));
    std::vector<std::array<float, 2>> out(positions.size() * inv_freq.size());
    dt.read_back(&out[0][0]);
    return out;
}

// ops::rope_neox_cached_from_array(x, table): one head, table = [sin, cos] pairs (rope.rs:70).
inline void rope_neox_cached_from_array(std::vector<float>& x, const std::vector<std::array<float, 2>>& table) {
    if (x.size() < table.size() * 2) throw Panic("assertion failed: x.len() >= table.len() * 2");
    Dev<float> dx(x.data(), x.size()), dt(&table[0][0], table.size() * 2);
    check(apk_qknorm_rope_neox(Gpu::get().ctx(), dx.ptr(), nullptr, nullptr, nullptr, dt.ptr(), 1, 1, 0, x.size(), table.size() * 2,
                               0.0f, APK_F32));
    dx.read_back(x.data());
}

// ops::add_assign_slice(a, b): a += b (blas.rs:105); a shorter or longer b panics.
inline void add_assign_slice(std::vector<float>& a, const std::vector<float>& b) {
    if (a.size() != b.size()) throw Panic("assertion `left == right` failed: a.len() == b.len()");
    Dev<float> da(a.data(), a.size()), db(b.data(), b.size());
    check(apk_add_assign(Gpu::get().ctx(), da.ptr(), db.ptr(), a.size(), APK_F32));
    da.read_back(a.data());
}

// ops::add_scaled_slice(dst, src, scale): dst = fma(src, scale, dst) (blas.rs:25-102); a shorter or longer src panics
// (ops/mod.rs:403-408).
inline void add_scaled_slice(std::vector<float>& dst, const std::vector<float>& src, float scale) {
    if (dst.size() != src.size()) throw Panic("assertion `left == right` failed: dst.len() == src.len()");
    Dev<float> dd(dst.data(), dst.size()), ds(src.data(), src.size());
    check(apk_add_scaled(Gpu::get().ctx(), dd.ptr(), ds.ptr(), dst.size(), scale, APK_F32));
    dd.read_back(dst.data());
}

// add_bias_rows(rows, bias) (model/loader.rs:519-523): every whole row of bias.len() elements gets the bias; what is
// left of a partial last row is untouched (chunks_exact_mut).
inline void add_bias_rows(std::vector<float>& rows, const std::vector<float>& bias) {
    if (bias.empty()) throw Panic("chunk size must be non-zero");
    const size_t n = bias.size(), whole = rows.size() / n;
    if (whole == 0) return;
    Dev<float> dx(rows.data(), whole * n), db(bias.data(), n);
    check(apk_add_bias_rows(Gpu::get().ctx(), dx.ptr(), db.ptr(), whole, n, APK_F32));
    dx.read_back(rows.data());
}

// ops::softmax(x) in place (activation.rs:5).
inline void softmax(std::vector<float>& x) {
    Dev<float> dx(x.data(), x.size());
    check(apk_softmax_rows(Gpu::get().ctx(), dx.ptr(), 1, x.size()));
    dx.read_back(x.data());
}

// ops::rope_norm_cached_from_array(x, table): adjacent pairs (2i, 2i+1) rotate (rope.rs:52).
inline void rope_norm_cached_from_array(std::vector<float>& x, const std::vector<std::array<float, 2>>& table) {
    if (x.size() < table.size() * 2) throw Panic("assertion failed: x.len() >= table.len() * 2");
    Dev<float> dx(x.data(), x.size()), dt(&table[0][0], table.size() * 2);
    check(apk_qknorm_rope_norm(Gpu::get().ctx(), dx.ptr(), nullptr, nullptr, nullptr, dt.ptr(), 1, 1, 0, x.size(), table.size() * 2,
                               0.0f, APK_F32));
    dx.read_back(x.data());
}

// The QK-norm + RoPE loop of run_cpu_attention_from_qkv (attention.rs:131-165) over rows of q and k.
inline void qknorm_rope_rows(std::vector<float>& q, std::vector<float>& k, const std::vector<float>* q_norm,
                             const std::vector<float>* k_norm, const std::vector<std::array<float, 2>>& rope_flat, size_t rows,
                             size_t n_q, size_t n_kv, size_t head_dim, float eps) {
    if (q.size() != rows * n_q * head_dim || k.size() != rows * n_kv * head_dim || rope_flat.size() != rows * head_dim / 2)
        throw Panic("qknorm_rope_rows: slice lengths");
    Dev<float> dq(q.data(), q.size()), dk(k.data(), k.size()), dt(&rope_flat[0][0], rope_flat.size() * 2);
    Dev<float> dqw(q_norm ? q_norm->data() : nullptr, head_dim), dkw(k_norm ? k_norm->data() : nullptr, head_dim);
    check(apk_qknorm_rope_neox(Gpu::get().ctx(), dq.ptr(), dk.ptr(), q_norm ? dqw.ptr() : nullptr, k_norm ? dkw.ptr() : nullptr,
                               dt.ptr(), rows, n_q, n_kv, head_dim, head_dim, eps, APK_F32));
    dq.read_back(q.data());
    dk.read_back(k.data());
}

// ops::swiglu(gate, up): gate = silu(gate) * up (activation.rs:57).
inline void swiglu(std::vector<float>& gate, const std::vector<float>& up) {
    if (gate.size() != up.size()) throw Panic("assertion failed: gate.len() == up.len()");
    Dev<float> dg(gate.data(), gate.size()), du(up.data(), up.size());
    check(apk_swiglu(Gpu::get().ctx(), dg.ptr(), du.ptr(), gate.size(), APK_F32));
    dg.read_back(gate.data());
}

// ops::geglu_tanh(gate, up): gate = gelu_tanh(gate) * up (activation.rs:44-51).
inline void geglu_tanh(std::vector<float>& gate, const std::vector<float>& up) {
    if (gate.size() != up.size()) throw Panic("assertion failed: gate.len() == up.len()");
    Dev<float> dg(gate.data(), gate.size()), du(up.data(), up.size());
    check(apk_geglu_tanh(Gpu::get().ctx(), dg.ptr(), du.ptr(), gate.size(), APK_F32));
    dg.read_back(gate.data());
}

}  // namespace ops

// QuantMat::{new,row,row_into} (quantmat/mod.rs:39-89): a quantised matrix whose rows are the embedding rows.
class QuantMat {
  public:
    QuantMat(const std::vector<uint8_t>& data, GgmlType ty, size_t n_out, size_t n_in) : ty_((int)ty), n_out_(n_out), n_in_(n_in) {
        const size_t rb = apk_row_bytes(ty_, n_in);
        if (ty_ < 0 || ty_ > 9) throw Error("unsupported ggml type");
        if (rb == 0) throw Error("row length is not a whole number of blocks");
        if (rb * n_out != data.size()) throw Error("byte count does not match n_out x n_in");
        dev_.reset(new Dev<uint8_t>(data.data(), data.size()));
        table_ = dev_->ptr();
    }
    // QuantMat::new over a borrowed slice of the model file (quantmat/mod.rs:39-66: `data: &'a [u8]`).  Bytes inside
    // an attached mapping are used where they already are on the device (resident() is true, nothing is copied) and
    // are named by their host address, resolved again at every call (resolve_w, gpu/cuda/runtime/select.rs:80-84):
    // the QuantMat takes no owner, so after the mapping's last detach every call throws Declined and launches nothing.
    // A slice of foreign memory -- the same bytes on the heap, say -- gets a device copy of its own.
    QuantMat(const uint8_t* data, size_t bytes, GgmlType ty, size_t n_out, size_t n_in) : ty_((int)ty), n_out_(n_out), n_in_(n_in) {
        const size_t rb = apk_row_bytes(ty_, n_in);
        if (ty_ < 0 || ty_ > 9) throw Error("unsupported ggml type");
        if (rb == 0) throw Error("row length is not a whole number of blocks");
        if (rb * n_out != bytes) throw Error("byte count does not match n_out x n_in");
        if (gpu::resolve(data, bytes)) {
            host_ = data;
            host_bytes_ = bytes;
        } else {
            dev_.reset(new Dev<uint8_t>(data, bytes));
            table_ = dev_->ptr();
        }
    }
    bool resident() const { return !dev_; }  // the table lives inside an attached mapping
    std::vector<float> row(size_t j) const {
        std::vector<float> out(n_in_);
        row_into(j, out);
        return out;
    }
    void row_into(size_t j, std::vector<float>& dst) const {
        if (j >= n_out_) throw Error("row " + std::to_string(j) + " out of " + std::to_string(n_out_));
        if (dst.size() != n_in_) throw Error("row_into destination has the wrong length");
        const uint32_t id = (uint32_t)j;
        Dev<float> dout(n_in_);
        check(apk_embed_rows_host_ids(Gpu::get().ctx(), ty_, table(), n_out_, n_in_, &id, 1, dout.ptr(), APK_F32));
        dout.read_back(dst.data());
    }
    // rows [row0, row0 + count) as f32, one launch, no id list (the same rows as row_into in a loop)
    std::vector<float> dequant_rows(size_t row0, size_t count) const {
        std::vector<float> out(count * n_in_);
        if (count == 0) return out;
        Dev<float> dout(out.size());
        check(apk_dequant_rows(Gpu::get().ctx(), ty_, table(), n_out_, n_in_, row0, count, dout.ptr(), APK_F32));
        dout.read_back(out.data());
        return out;
    }

  private:
    // the table's device address for this call: its own copy, or wherever the attached mapping holds it now
    const void* table() const {
        if (!host_) return table_;
        void* dev = nullptr;
        check(apk_resolve(Gpu::get().ctx(), host_, host_bytes_, &dev));  // Declined once the mapping is detached
        return dev;
    }
    int ty_;
    size_t n_out_, n_in_;
    std::unique_ptr<Dev<uint8_t>> dev_;  // the table's own device copy, when it is not inside an attached mapping
    const void* table_ = nullptr;
    const uint8_t* host_ = nullptr;      // a borrowed slice inside an attached mapping (resolved per call)
    size_t host_bytes_ = 0;
};

// model::route_gated(logits, k, gating, norm, scale, bias) -> best-first (expert, weight) (moe.rs:601-616).
inline std::vector<std::pair<size_t, float>> route_gated(const std::vector<float>& logits, size_t k, Gating gating, bool norm,
                                                          float scale, const std::vector<float>* bias) {
    k = k < logits.size() ? k : logits.size();
    if (k == 0) return {};
    Dev<float> dl(logits.data(), logits.size()), dw(k), db(bias ? bias->data() : nullptr, logits.size());
    Dev<uint32_t> di(k);
    check(apk_route_topk(Gpu::get().ctx(), dl.ptr(), bias ? db.ptr() : nullptr, 1, logits.size(), k, norm ? 1 : 0, scale,
                         gating == Gating::Sigmoid ? 1 : 0, di.ptr(), dw.ptr()));
    std::vector<uint32_t> ids(k);
    std::vector<float> w(k);
    di.read_back(ids.data());
    dw.read_back(w.data());
    std::vector<std::pair<size_t, float>> out;
    for (size_t i = 0; i < k; i++) out.emplace_back(ids[i], w[i]);
    return out;
}

// model::route(probs, k) (moe.rs:623-658): the top k of an already softmaxed row, renormalised to sum to 1, best first.
inline std::vector<std::pair<size_t, float>> route(const std::vector<float>& probs, size_t k) {
    k = k < probs.size() ? k : probs.size();
    if (k == 0) return {};
    Dev<float> dp(probs.data(), probs.size()), dw(k);
    Dev<uint32_t> di(k);
    check(apk_route_topk(Gpu::get().ctx(), dp.ptr(), nullptr, 1, probs.size(), k, 1, 1.0f, 2, di.ptr(), dw.ptr()));
    std::vector<uint32_t> ids(k);
    std::vector<float> w(k);
    di.read_back(ids.data());
    dw.read_back(w.data());
    std::vector<std::pair<size_t, float>> out;
    for (size_t i = 0; i < k; i++) out.emplace_back(ids[i], w[i]);
    return out;
}

// The batched router of Ffn::moe_batch (moe.rs:204-227): route_gated_into_slice for every row of
// logits [rows][n_expert]; ids and w are [rows][k], best first.
struct Routed {
    size_t rows = 0, k = 0;
    std::vector<uint32_t> ids;
    std::vector<float> w;
};
inline Routed route_rows(const std::vector<float>& logits, size_t n_expert, size_t k, Gating gating, bool norm, float scale,
                         const std::vector<float>* bias) {
    if (n_expert == 0 || logits.size() % n_expert) throw Panic("logits is not rows x n_expert");
    if (bias && bias->size() != n_expert) throw Panic("bias length is not n_expert");
    Routed r;
    r.rows = logits.size() / n_expert;
    r.k = k < n_expert ? k : n_expert;
    r.ids.resize(r.rows * r.k);
    r.w.resize(r.rows * r.k);
    if (r.rows == 0 || r.k == 0) return r;
    Dev<float> dl(logits.data(), logits.size()), dw(r.w.size()), db(bias ? bias->data() : nullptr, n_expert);
    Dev<uint32_t> di(r.ids.size());
    check(apk_route_topk(Gpu::get().ctx(), dl.ptr(), bias ? db.ptr() : nullptr, r.rows, n_expert, r.k, norm ? 1 : 0, scale,
                         gating == Gating::Sigmoid ? 1 : 0, di.ptr(), dw.ptr()));
    di.read_back(r.ids.data());
    dw.read_back(r.w.data());
    return r;
}

// groups / used / table / tok of Ffn::moe_batch and the per-token hit lists of its combine
// (moe.rs:229-271, :298-309), i.e. GroupedFfnReq.{groups, tok, total_rows} and
// GroupedCombine.{tok_off, hit_row, hit_w} (gpu/types.rs:429-467).
struct Grouped {
    std::vector<std::array<uint32_t, 3>> groups;  // [expert, row0, rows] of the experts that were hit, ascending
    std::vector<uint32_t> tok;                    // source token of each flat row
    std::vector<uint32_t> tok_off, hit_row;       // CSR: token t's hits are [tok_off[t], tok_off[t+1])
    std::vector<float> hit_w;
    size_t total_rows = 0;
};
inline Grouped moe_group(const Routed& r, size_t n_expert) {
    Grouped g;
    const size_t total = r.rows * r.k;
    g.total_rows = total;
    g.tok_off.assign(r.rows + 1, 0);
    if (total == 0) return g;
    Dev<uint32_t> di(r.ids.data(), total), dtable(n_expert * 3), dn(1), dtok(total), doff(r.rows + 1), dhit(total);
    Dev<float> dw(r.w.data(), total), dhw(total);
    check(apk_moe_permute(Gpu::get().ctx(), di.ptr(), dw.ptr(), r.rows, r.k, n_expert, dtable.ptr(), dn.ptr(), dtok.ptr(),
                          doff.ptr(), dhit.ptr(), dhw.ptr()));
    uint32_t faults = 0;
    check(apk_take_faults(Gpu::get().ctx(), &faults));
    if (faults) throw Panic("expert id out of range");  // groups[e] would index out of bounds
    uint32_t n_used = 0;
    dn.read_back(&n_used);
    std::vector<uint32_t> table(n_expert * 3);
    dtable.read_back(table.data());
    for (uint32_t i = 0; i < n_used; i++) g.groups.push_back({table[3 * i], table[3 * i + 1], table[3 * i + 2]});
    g.tok.resize(total);
    g.hit_row.resize(total);
    g.hit_w.resize(total);
    dtok.read_back(g.tok.data());
    doff.read_back(g.tok_off.data());
    dhit.read_back(g.hit_row.data());
    dhw.read_back(g.hit_w.data());
    return g;
}

// The gathered expert activations xe[r] = x[tok[r]] (moe.rs:348-352), produced from the token side.
inline std::vector<float> gather_rows(const std::vector<float>& x, size_t hidden, const Grouped& g, size_t k) {
    if (hidden == 0 || x.size() % hidden) throw Panic("x is not rows x hidden");
    const size_t rows = x.size() / hidden;
    if (rows * k != g.total_rows) throw Panic("grouping does not belong to these rows");
    std::vector<float> xe(g.total_rows * hidden);
    if (xe.empty()) return xe;
    Dev<float> dx(x.data(), x.size()), dxe(xe.size());
    Dev<uint32_t> dhit(g.hit_row.data(), g.hit_row.size());
    check(apk_scatter_rows(Gpu::get().ctx(), dx.ptr(), dhit.ptr(), rows, k, g.total_rows, hidden, dxe.ptr(), APK_F32));
    dxe.read_back(xe.data());
    return xe;
}

// The combine of Ffn::moe_batch (moe.rs:298-333: per token, add_scaled_slice over its hits in order),
// the residual add (decode.rs:775) and, when next_norm is given, the next layer's rmsnorm_rows_into
// (prefill.rs:308-314) in one pass: x += sum; h = rmsnorm(x) * next_norm.
inline void moe_combine_add_rmsnorm(std::vector<float>& x, const std::vector<float>& flat, size_t hidden, const Grouped& g,
                                    std::vector<float>* h, const std::vector<float>* next_norm, float eps) {
    if (hidden == 0 || x.size() % hidden || flat.size() != g.total_rows * hidden) throw Panic("shape mismatch");
    const size_t rows = x.size() / hidden;
    if (g.tok_off.size() != rows + 1) throw Panic("grouping does not belong to these rows");
    if (h && (!next_norm || next_norm->size() != hidden || h->size() < x.size())) throw Panic("next norm shape mismatch");
    if (rows == 0) return;
    Dev<float> dx(x.data(), x.size()), dflat(flat.data(), flat.size()), dhw(g.hit_w.data(), g.hit_w.size()), dh(h ? x.size() : 1),
        dgamma(h ? next_norm->data() : nullptr, h ? hidden : 1);
    Dev<uint32_t> doff(g.tok_off.data(), g.tok_off.size()), dhit(g.hit_row.data(), g.hit_row.size());
    check(apk_moe_combine_add_rmsnorm(Gpu::get().ctx(), dx.ptr(), dflat.ptr(), doff.ptr(), dhit.ptr(), dhw.ptr(), g.total_rows,
                                      h ? dh.ptr() : nullptr, h ? dgamma.ptr() : nullptr, hidden, rows, eps, APK_F32));
    dx.read_back(x.data());
    if (h) dh.read_back(h->data());
}

// The greedy pick of forward_greedy (decode.rs:628-630): max_by(total_cmp), i.e. the LAST maximum.
inline uint32_t argmax(const std::vector<float>& logits) {
    if (logits.empty()) return 0;  // unwrap_or(0)
    Dev<float> dl(logits.data(), logits.size());
    Dev<uint32_t> dout(1);
    check(apk_argmax_rows(Gpu::get().ctx(), dl.ptr(), 1, logits.size(), dout.ptr()));
    uint32_t out = 0;
    dout.read_back(&out);
    return out;
}

// One layer's K and V planes of the cache, [capacity][kv_dim] f16 each (kv.rs:682-697), on the device.
class KvLayer {
  public:
    KvLayer(size_t capacity, size_t kv_dim) : capacity_(capacity), kv_dim_(kv_dim), k_(capacity * kv_dim), v_(capacity * kv_dim) {}
    // The attention prologue of a chunk (attention.rs:131-200): per-head rmsnorm + NeoX rotation of q and k
    // in place, then KvCache::store_at(layer, pos[r], k_row, v_row) for every row -- one launch.
    void qknorm_rope_store(std::vector<float>& q, std::vector<float>& k, const std::vector<float>& v, const std::vector<float>* q_norm,
                           const std::vector<float>* k_norm, const std::vector<std::array<float, 2>>& rope,
                           const std::vector<uint32_t>& pos, size_t n_q, size_t n_kv, size_t head_dim, float eps) {
        const size_t rows = pos.size();
        if (n_kv * head_dim != kv_dim_ || k.size() != rows * kv_dim_ || v.size() != k.size() || q.size() != rows * n_q * head_dim)
            throw Panic("k / v rows are not kv_dim wide");  // assert_eq!(k.len(), self.kv_dim)
        if (rope.size() != rows * head_dim / 2) throw Panic("rope table does not cover the rows");
        for (uint32_t p : pos)
            if (p >= capacity_) throw Panic("position " + std::to_string(p) + " past capacity " + std::to_string(capacity_));
        if (rows == 0) return;
        Dev<float> dq(q.data(), q.size()), dk(k.data(), k.size()), dv(v.data(), v.size()), drope(&rope[0][0], rope.size() * 2),
            dqw(q_norm ? q_norm->data() : nullptr, head_dim), dkw(k_norm ? k_norm->data() : nullptr, head_dim);
        Dev<uint32_t> dpos(pos.data(), rows);
        check(apk_qknorm_rope_kv_store(Gpu::get().ctx(), dq.ptr(), dk.ptr(), dv.ptr(), q_norm ? dqw.ptr() : nullptr,
                                       k_norm ? dkw.ptr() : nullptr, drope.ptr(), dpos.ptr(), k_.ptr(), v_.ptr(), capacity_, rows, n_q,
                                       n_kv, head_dim, head_dim, eps, APK_F32));
        dq.read_back(q.data());
        dk.read_back(k.data());
    }
    // the stored f16 bits of one position
    std::vector<uint16_t> k_row(size_t pos) const { return row(k_, pos); }
    std::vector<uint16_t> v_row(size_t pos) const { return row(v_, pos); }

  private:
    std::vector<uint16_t> row(const Dev<uint16_t>& plane, size_t pos) const {
        if (pos >= capacity_) throw Panic("position past capacity");
        std::vector<uint16_t> out(kv_dim_);
        check(apk_d2h(Gpu::get().ctx(), out.data(), plane.ptr() + pos * kv_dim_, kv_dim_ * 2));
        check(apk_sync(Gpu::get().ctx()));
        return out;
    }
    size_t capacity_, kv_dim_;
    Dev<uint16_t> k_, v_;
};

}  // namespace allpaka_backend

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

// ops::rope_inv_freq / rope_sin_cos (rope.rs:8-22) stay host-side one-liners in the reference; the table rows
// for a batch of positions can be built on the device:
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
    }
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
        check(apk_embed_rows_host_ids(Gpu::get().ctx(), ty_, dev_->ptr(), n_out_, n_in_, &id, 1, dout.ptr(), APK_F32));
        dout.read_back(dst.data());
    }
    // rows [row0, row0 + count) as f32, one launch, no id list (the same rows as row_into in a loop)
    std::vector<float> dequant_rows(size_t row0, size_t count) const {
        std::vector<float> out(count * n_in_);
        if (count == 0) return out;
        Dev<float> dout(out.size());
        check(apk_dequant_rows(Gpu::get().ctx(), ty_, dev_->ptr(), n_out_, n_in_, row0, count, dout.ptr(), APK_F32));
        dout.read_back(out.data());
        return out;
    }

  private:
    int ty_;
    size_t n_out_, n_in_;
    std::unique_ptr<Dev<uint8_t>> dev_;
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

}  // namespace allpaka_backend

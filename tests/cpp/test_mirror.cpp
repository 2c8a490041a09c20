// The reference's own unit tests for this path, re-expressed against the C++ host mirror
// (include/allpaka_backend.hpp) so that they run on the MI355X through the C ABI.
// Each test names the reference test it follows (crates/allpaka-backend/src/ops/mod.rs unless noted).
#include <cmath>
#include <cstdio>
#include <functional>

#include "allpaka_backend.hpp"

using namespace allpaka_backend;
static int failures = 0;
#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);  \
            failures++;                                                      \
        }                                                                    \
    } while (0)
static bool close(float a, float b) { return std::fabs(a - b) < 1e-5f * (1.0f + std::fabs(b)); }  // ops/mod.rs:25-27
template <typename E> static bool throws(std::function<void()> f) {
    try { f(); } catch (const E&) { return true; } catch (...) { return false; }
    return false;
}
static float silu(float x) { return x / (1.0f + std::exp(-x)); }

static void rmsnorm_normalises_to_unit_rms_before_the_weight() {  // :119-128
    std::vector<float> x = {3.0f, -4.0f, 12.0f, 0.0f}, w(4, 1.0f);
    ops::rmsnorm(x, w, 0.0f);
    float ss = 0;
    for (float v : x) ss += v * v;
    CHECK(close(std::sqrt(ss / 4.0f), 1.0f));
    CHECK(x[0] > 0.0f && x[1] < 0.0f && x[3] == 0.0f);
}
static void rmsnorm_applies_the_weight_per_channel() {  // :130-135 (a 2-element row: the element-wise path)
    std::vector<float> x = {1.0f, 1.0f};
    ops::rmsnorm(x, {2.0f, 3.0f}, 0.0f);
    CHECK(close(x[0], 2.0f) && close(x[1], 3.0f));
}
static void rmsnorm_eps_keeps_zero_input_finite() {  // :139-144
    std::vector<float> x(8, 0.0f);
    ops::rmsnorm(x, std::vector<float>(8, 1.0f), 1e-5f);
    for (float v : x) CHECK(std::isfinite(v));
}
static void rmsnorm_rows_into_rejects_a_short_destination() {  // :412-419
    const size_t n = 1024;
    std::vector<float> src(64 * n, 1.0f), dst(8 * n, 0.0f), w(n, 1.0f);
    bool ok = false;
    try { ops::rmsnorm_rows_into(dst, src, w, 1e-6f); } catch (const Panic& p) { ok = std::string(p.what()) == "dst holds fewer rows than src"; }
    CHECK(ok);
    CHECK(throws<Panic>([] { std::vector<float> x(4), w(3); ops::rmsnorm(x, w, 0.0f); }));
}
static void add_assign_then_norm_matches_the_two_ops() {  // decode.rs:584 then :764
    const size_t n = 1024, rows = 3;
    std::vector<float> a(rows * n), b(rows * n), h(rows * n), w(n);
    for (size_t i = 0; i < a.size(); i++) { a[i] = std::sin(0.1f * i); b[i] = std::cos(0.07f * i); }
    for (size_t i = 0; i < n; i++) w[i] = 1.0f + 0.001f * i;
    std::vector<float> sum(a);
    for (size_t i = 0; i < a.size(); i++) sum[i] = a[i] + b[i];
    ops::add_assign_then_rmsnorm_into(a, b, h, w, 1e-6f);
    for (size_t i = 0; i < a.size(); i++) CHECK(a[i] == sum[i]);
    std::vector<float> want(rows * n);
    ops::rmsnorm_rows_into(want, sum, w, 1e-6f);
    for (size_t i = 0; i < h.size(); i++) CHECK(h[i] == want[i]);
    CHECK(throws<Panic>([] { std::vector<float> a(64), b(8), h(64), w(64); ops::add_assign_then_rmsnorm_into(a, b, h, w, 0.0f); }));  // :396-401
}
static void swiglu_is_silu_of_gate_times_up() {  // :172-185, silu fixed points :163-170
    std::vector<float> gate, up;
    for (int i = -25; i < 26; i++) gate.push_back(i * 0.7f);
    for (size_t i = 0; i < gate.size(); i++) up.push_back(i * 0.5f - 3.0f);
    std::vector<float> orig(gate);
    ops::swiglu(gate, up);
    for (size_t i = 0; i < gate.size(); i++) CHECK(close(gate[i], silu(orig[i]) * up[i]));
    std::vector<float> g = {0.0f, 1.0f, -20.0f, 20.0f}, u(4, 1.0f);
    ops::swiglu(g, u);
    CHECK(g[0] == 0.0f && close(g[1], 1.0f / (1.0f + std::exp(-1.0f))) && std::fabs(g[2]) < 1e-7f && close(g[3], 20.0f));
    CHECK(throws<Panic>([] { std::vector<float> g(4), u(3); ops::swiglu(g, u); }));
}
static void softmax_sums_to_one_and_survives_huge_logits() {  // ops/mod.rs:147-161
    std::vector<float> x = {1.0f, 3.0f, 2.0f};
    ops::softmax(x);
    CHECK(close(x[0] + x[1] + x[2], 1.0f) && x[1] > x[2] && x[2] > x[0]);
    std::vector<float> y = {1000.0f, 999.0f};
    ops::softmax(y);
    CHECK(std::isfinite(y[0]) && std::isfinite(y[1]) && close(y[0] + y[1], 1.0f));
}
static void add_assign_slice_adds_and_rejects_length_mismatch() {  // ops/mod.rs:394-408
    std::vector<float> a = {1.0f, 2.0f, 3.0f, 4.0f, 5.0f}, b = {0.5f, -2.0f, 10.0f, 0.25f, -5.0f};
    ops::add_assign_slice(a, b);
    CHECK((a == std::vector<float>{1.5f, 0.0f, 13.0f, 4.25f, 0.0f}));
    CHECK(throws<Panic>([] { std::vector<float> a(8), b(7); ops::add_assign_slice(a, b); }));
}
static std::vector<std::array<float, 2>> table_for(uint32_t pos, size_t head_dim, float base) {  // rope.rs:8-22
    std::vector<std::array<float, 2>> t(head_dim / 2);
    for (size_t i = 0; i < head_dim / 2; i++) {
        const float a = (float)pos * std::pow(base, -2.0f * (float)i / (float)head_dim);
        t[i] = {std::sin(a), std::cos(a)};
    }
    return t;
}
static void rope_is_norm_preserving_and_identity_at_position_zero() {  // :188-202 (head of 128)
    std::vector<float> orig(128);
    for (size_t i = 0; i < 128; i++) orig[i] = (float)i - 63.5f;
    std::vector<float> x(orig);
    ops::rope_neox_cached_from_array(x, table_for(0, 128, 10000.0f));
    CHECK(x == orig);
    ops::rope_neox_cached_from_array(x, table_for(17, 128, 10000.0f));
    float n0 = 0, n1 = 0;
    for (size_t i = 0; i < 128; i++) { n0 += orig[i] * orig[i]; n1 += x[i] * x[i]; }
    CHECK(close(n0, n1) && x != orig);
}
static void rope_neox_pairs_split_channels() {  // :206-221
    std::vector<float> x(128, 0.0f);
    x[0] = 1.0f;
    ops::rope_neox_cached_from_array(x, table_for(1, 128, 10000.0f));
    CHECK(close(x[64], std::sin(1.0f)) && x[1] == 0.0f);
    // adjacent-pair style: channel 0 pairs with channel 1 (rope.rs:90-101)
    std::vector<float> y(128, 0.0f);
    y[0] = 1.0f;
    ops::rope_norm_cached_from_array(y, table_for(1, 128, 10000.0f));
    CHECK(close(y[1], std::sin(1.0f)) && y[64] == 0.0f);
}
static void partial_rotary_rotates_the_head_and_passes_the_tail() {  // :367-391 (12-wide head, 8 rotating channels)
    std::vector<float> orig(12);
    for (size_t i = 0; i < 12; i++) orig[i] = 0.25f * (float)i - 1.0f;
    auto table = table_for(5, 8, 10000.0f);
    std::vector<float> a(orig), b(orig);
    ops::rope_neox_cached_from_array(a, table);
    ops::rope_norm_cached_from_array(b, table);
    for (size_t i = 8; i < 12; i++) CHECK(a[i] == orig[i] && b[i] == orig[i]);
    // the rotating channels are those of an 8-wide head on its own
    std::vector<float> a8(orig.begin(), orig.begin() + 8), b8(a8);
    ops::rope_neox_cached_from_array(a8, table);
    ops::rope_norm_cached_from_array(b8, table);
    for (size_t i = 0; i < 8; i++) CHECK(a[i] == a8[i] && b[i] == b8[i]);
    CHECK(a8 != b8);
    // a table longer than the head is the reference's assertion
    CHECK(throws<Panic>([] { std::vector<float> x(8, 1.0f); ops::rope_neox_cached_from_array(x, table_for(1, 16, 10000.0f)); }));
}
static void device_rope_rows_match_the_host_table() {  // session.rs:34-50
    std::vector<float> inv(64);
    for (size_t i = 0; i < 64; i++) inv[i] = std::pow(1e6f, -2.0f * (float)i / 128.0f);
    auto rows = ops::rope_sin_cos_rows({0, 1, 511, 32767}, inv);
    const uint32_t pos[4] = {0, 1, 511, 32767};
    for (int r = 0; r < 4; r++) {
        auto want = table_for(pos[r], 128, 1e6f);
        for (size_t i = 0; i < 64; i++) CHECK(std::fabs(rows[r * 64 + i][0] - want[i][0]) < 3e-7f && std::fabs(rows[r * 64 + i][1] - want[i][1]) < 3e-7f);
    }
}
static void q8_0_is_scale_times_value() {  // crates/allpaka-gguf/src/dequant.rs:317-331 through QuantMat::row
    std::vector<uint8_t> block(34 * 2, 0);
    block[0] = 0x00; block[1] = 0x38;  // f16 0.5
    block[2] = 10; block[3] = (uint8_t)(int8_t)-20; block[33] = 127;
    block[34] = 0x00; block[35] = 0x3c;  // second block: scale 1.0
    QuantMat m(block, GgmlType::Q8_0, 1, 64);
    auto out = m.row(0);
    CHECK(out.size() == 64 && out[0] == 5.0f && out[1] == -10.0f && out[31] == 63.5f && out[2] == 0.0f);
    // quantmat/mod.rs:923-937
    CHECK(throws<Error>([&] { m.row(1); }));
    CHECK(throws<Error>([&] { QuantMat bad(block, GgmlType::Q8_0, 1, 48); }));
    CHECK(throws<Error>([&] { std::vector<float> d(32); m.row_into(0, d); }));
    // the same bytes as two rows of 32: a range of rows in one launch equals the rows one by one
    QuantMat m2(block, GgmlType::Q8_0, 2, 32);
    auto both = m2.dequant_rows(0, 2);
    CHECK(both.size() == 64 && both == out);
    auto second = m2.dequant_rows(1, 1);
    CHECK(second.size() == 32 && second == m2.row(1));
    CHECK(throws<Declined>([&] { m2.dequant_rows(1, 2); }));
}
static void route_picks_the_top_k_and_renormalises() {  // crates/allpaka-model/tests/gpu_eligible_forward.rs:88-97
    std::vector<float> logp = {std::log(0.1f), std::log(0.5f), std::log(0.15f), std::log(0.25f)};
    auto picked = route_gated(logp, 2, Gating::Softmax, true, 1.0f, nullptr);
    CHECK(picked.size() == 2 && picked[0].first == 1 && picked[1].first == 3);
    CHECK(std::fabs(picked[0].second - 2.0f / 3.0f) < 1e-6f && std::fabs(picked[1].second - 1.0f / 3.0f) < 1e-6f);
    // moe.rs:664-669 logits, k clamps to n, ties -> lower index
    std::vector<float> t(16, 0.0f);
    t[3] = t[9] = t[12] = 2.0f;
    t[5] = t[7] = 1.0f;
    auto p = route_gated(t, 4, Gating::Softmax, true, 1.0f, nullptr);
    CHECK(p.size() == 4 && p[0].first == 3 && p[1].first == 9 && p[2].first == 12 && p[3].first == 5);
    CHECK(route_gated({1.0f, 2.0f}, 8, Gating::Softmax, true, 1.0f, nullptr).size() == 2);
    CHECK(route_gated({1.0f, 2.0f}, 0, Gating::Softmax, true, 1.0f, nullptr).empty());
}

int main() {
    struct { const char* name; void (*fn)(); } tests[] = {
        {"rmsnorm_normalises_to_unit_rms_before_the_weight", rmsnorm_normalises_to_unit_rms_before_the_weight},
        {"rmsnorm_applies_the_weight_per_channel", rmsnorm_applies_the_weight_per_channel},
        {"rmsnorm_eps_keeps_zero_input_finite", rmsnorm_eps_keeps_zero_input_finite},
        {"rmsnorm_rows_into_rejects_a_short_destination", rmsnorm_rows_into_rejects_a_short_destination},
        {"add_assign_then_norm_matches_the_two_ops", add_assign_then_norm_matches_the_two_ops},
        {"swiglu_is_silu_of_gate_times_up", swiglu_is_silu_of_gate_times_up},
        {"softmax_sums_to_one_and_survives_huge_logits", softmax_sums_to_one_and_survives_huge_logits},
        {"add_assign_slice_adds_and_rejects_length_mismatch", add_assign_slice_adds_and_rejects_length_mismatch},
        {"rope_is_norm_preserving_and_identity_at_position_zero", rope_is_norm_preserving_and_identity_at_position_zero},
        {"rope_neox_pairs_split_channels", rope_neox_pairs_split_channels},
        {"partial_rotary_rotates_the_head_and_passes_the_tail", partial_rotary_rotates_the_head_and_passes_the_tail},
        {"device_rope_rows_match_the_host_table", device_rope_rows_match_the_host_table},
        {"q8_0_is_scale_times_value", q8_0_is_scale_times_value},
        {"route_picks_the_top_k_and_renormalises", route_picks_the_top_k_and_renormalises},
    };
    try {
        Gpu::get();
    } catch (const std::exception& e) {
        std::printf("no usable GPU: %s\n", e.what());
        return 77;
    }
    for (auto& t : tests) {
        const int before = failures;
        std::printf("test %s ... ", t.name);
        std::fflush(stdout);
        try {
            t.fn();
        } catch (const std::exception& e) {
            std::printf("\n  threw %s", e.what());
            failures++;
        }
        std::printf("%s\n", failures == before ? "ok" : "FAILED");
    }
    std::printf("%d failure(s)\n", failures);
    return failures ? 1 : 0;
}

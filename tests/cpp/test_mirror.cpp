// The reference's own unit tests for this path, re-expressed against the C++ host mirror
// (include/allpaka_backend.hpp) so that they run on the MI355X through the C ABI.
// Each test names the reference test it follows (crates/allpaka-backend/src/ops/mod.rs unless noted).
#include <cmath>
#include <cstdio>
#include <cstring>
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
static void sandwich_norm_matches_the_three_ops() {  // decode.rs:581-584, :771-775, then :762-764
    const size_t n = 2304, rows = 5;
    std::vector<float> a(rows * n), d(rows * n), h(rows * n), w(n), pw(n);
    for (size_t i = 0; i < a.size(); i++) { a[i] = std::sin(0.1f * i); d[i] = 3.0f * std::cos(0.07f * i); }
    for (size_t i = 0; i < n; i++) { w[i] = 1.0f + 0.001f * i; pw[i] = 0.5f + 0.0003f * i; }
    std::vector<float> nd(rows * n), sum(a), want(rows * n);
    ops::rmsnorm_rows_into(nd, d, pw, 1e-6f);
    for (size_t i = 0; i < a.size(); i++) sum[i] = a[i] + nd[i];
    ops::rmsnorm_rows_into(want, sum, w, 1e-6f);
    const std::vector<float> d0(d);
    ops::postnorm_add_assign_then_rmsnorm_into(a, d, pw, h, w, 1e-6f);
    for (size_t i = 0; i < a.size(); i++) CHECK(a[i] == sum[i] && d[i] == d0[i]);
    for (size_t i = 0; i < h.size(); i++) CHECK(h[i] == want[i]);
    CHECK(throws<Panic>([] { std::vector<float> a(64), d(64), pw(32), h(64), w(64); ops::postnorm_add_assign_then_rmsnorm_into(a, d, pw, h, w, 0.0f); }));
}
static void add_bias_rows_biases_every_whole_row() {  // loader.rs:519-523
    std::vector<float> x = {1, 2, 3, 4, 5, 6, 7, 8}, b = {10, 20, 30};
    ops::add_bias_rows(x, b);
    const std::vector<float> want = {11, 22, 33, 14, 25, 36, 7, 8};
    CHECK(x == want);
    std::vector<float> big(300 * 1024), bias(1024);
    for (size_t i = 0; i < big.size(); i++) big[i] = std::sin(0.01f * i);
    for (size_t i = 0; i < bias.size(); i++) bias[i] = 0.001f * i - 0.5f;
    std::vector<float> sum(big);
    for (size_t i = 0; i < big.size(); i++) sum[i] = big[i] + bias[i % 1024];
    ops::add_bias_rows(big, bias);
    CHECK(big == sum);
    CHECK(throws<Panic>([] { std::vector<float> x(4), b; ops::add_bias_rows(x, b); }));
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
static void geglu_tanh_is_the_tanh_gelu_of_gate_times_up() {  // activation.rs:44-51
    auto gelu = [](float x) { return 0.5f * x * (1.0f + std::tanh(0.7978846f * x * (1.0f + 0.044715f * x * x))); };
    std::vector<float> gate, up;
    for (int i = -40; i <= 40; i++) { gate.push_back(0.25f * (float)i); up.push_back(1.0f + 0.01f * (float)i); }
    std::vector<float> want(gate.size());
    for (size_t i = 0; i < gate.size(); i++) want[i] = gelu(gate[i]) * up[i];
    ops::geglu_tanh(gate, up);
    for (size_t i = 0; i < gate.size(); i++) CHECK(close(gate[i], want[i]));
    std::vector<float> z = {0.0f}, one = {3.0f};
    ops::geglu_tanh(z, one);
    CHECK(z[0] == 0.0f);  // gelu(0) = 0
    std::vector<float> big = {30.0f, -30.0f}, u2 = {2.0f, 2.0f};
    ops::geglu_tanh(big, u2);
    CHECK(big[0] == 60.0f && std::fabs(big[1]) < 1e-20f);  // identity far right, zero far left
    CHECK(throws<Panic>([] { std::vector<float> a(4), b(3); ops::geglu_tanh(a, b); }));
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
static void add_scaled_slice_is_one_fma_and_rejects_length_mismatch() {  // blas.rs:25-102, ops/mod.rs:403-408
    std::vector<float> a = {1.0f, 2.0f, -3.0f, 0.1f}, b = {0.5f, -2.0f, 10.0f, 0.3f};
    ops::add_scaled_slice(a, b, 0.7f);
    for (size_t i = 0; i < a.size(); i++) {
        const float d0[] = {1.0f, 2.0f, -3.0f, 0.1f};
        CHECK(a[i] == std::fmaf(b[i], 0.7f, d0[i]));
    }
    CHECK(throws<Panic>([] { std::vector<float> a(64), b(8); ops::add_scaled_slice(a, b, 2.0f); }));
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
// The same bytes opened twice (crates/allpaka-backend/tests/gpu_parity.rs:139-208): inside an attached mapping the table is
// used where it is on the device; as a heap copy it is foreign memory and gets a device copy of its own.  Owners are
// counted per (address, length) (gpu/cuda/runtime/device.rs:588-621).
static void weights_are_named_by_host_address_inside_an_attached_mapping() {
    std::vector<uint8_t> file(64 + 34 * 4 + 32, 0);  // a "model file": 64 bytes of header, a 2 x 64 Q8_0 table
    uint8_t* table = file.data() + 64;
    for (int b = 0; b < 4; b++) {
        table[34 * b] = 0x00; table[34 * b + 1] = 0x38;  // scale 0.5
        for (int i = 0; i < 32; i++) table[34 * b + 2 + i] = (uint8_t)(int8_t)(b * 32 + i - 60);
    }
    CHECK(gpu::resolve(table, 34 * 4) == nullptr && gpu::owners(file.data(), file.size()) == 0);
    CHECK(gpu::attach(file.data(), file.size()) && gpu::attach(file.data(), file.size()));
    CHECK(gpu::owners(file.data(), file.size()) == 2);
    CHECK(gpu::attach(table, 34) && gpu::owners(file.data(), file.size()) == 2);  // inside: no copy, no count
    CHECK(!gpu::attach(file.data() + 8, file.size()));                             // runs off the end: declined
    QuantMat resident(table, 34 * 4, GgmlType::Q8_0, 2, 64);
    std::vector<uint8_t> heap(table, table + 34 * 4);
    QuantMat foreign(heap.data(), heap.size(), GgmlType::Q8_0, 2, 64);
    CHECK(resident.resident() && !foreign.resident());
    CHECK(resident.row(1) == foreign.row(1) && resident.row(0)[0] == 0.5f * -60.0f && resident.row(1)[63] == 0.5f * 67.0f);
    CHECK(throws<Error>([&] { QuantMat bad(table, 34 * 4 - 1, GgmlType::Q8_0, 2, 64); }));
    CHECK((const uint8_t*)gpu::resolve(table + 34, 34) - (const uint8_t*)gpu::resolve(file.data(), 1) == 64 + 34);
    CHECK(gpu::resolve(table, file.size()) == nullptr);  // runs off the end of the mapping
    CHECK(gpu::detach(file.data(), file.size()));
    CHECK(gpu::owners(file.data(), file.size()) == 1 && gpu::resolve(table, 34) != nullptr);
    CHECK(gpu::detach(file.data(), file.size()));
    CHECK(gpu::owners(file.data(), file.size()) == 0 && gpu::resolve(table, 34) == nullptr);
    CHECK(!gpu::detach(file.data(), file.size()));  // silent when nothing is attached
    // the borrowed QuantMat holds no owner: with the mapping gone it declines instead of reading freed memory,
    // and a new file attached at the same address is what it reads next
    CHECK(throws<Declined>([&] { resident.row(1); }));
    CHECK(throws<Declined>([&] { resident.dequant_rows(0, 2); }));
    for (int i = 0; i < 32; i++) table[34 * 2 + 2 + i] = (uint8_t)(int8_t)(i - 7);  // row 1, first block: new quants
    CHECK(gpu::attach(file.data(), file.size()));
    CHECK(resident.row(1)[0] == 0.5f * -7.0f && resident.row(1)[31] == 0.5f * 24.0f);
    CHECK(gpu::detach(file.data(), file.size()));
}
static void route_picks_the_top_k_and_renormalises() {  // crates/allpaka-model/tests/gpu_eligible_forward.rs:88-97
    // the test as the reference writes it: route(&[0.1, 0.5, 0.15, 0.25], 2) on probabilities
    auto direct = route({0.1f, 0.5f, 0.15f, 0.25f}, 2);
    CHECK(direct.size() == 2 && direct[0].first == 1 && direct[1].first == 3);
    CHECK(direct[0].second == 0.5f / (0.5f + 0.25f) && direct[1].second == 0.25f / (0.5f + 0.25f));
    CHECK(route({0.25f, 0.25f}, 5).size() == 2 && route({}, 2).empty());
    auto flat = route({0.0f, 0.0f, 0.0f}, 2);  // nothing to renormalise by: 1 / k each, lower index first
    CHECK(flat.size() == 2 && flat[0].first == 0 && flat[1].first == 1 && flat[0].second == 0.5f);
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

// ---- the MoE grouping, combine, greedy pick and cache store, against the reference's CPU algorithm restated here
static Routed picks(size_t rows, size_t k, std::vector<uint32_t> ids, std::vector<float> w) {
    Routed r;
    r.rows = rows; r.k = k; r.ids = std::move(ids); r.w = std::move(w);
    return r;
}
static Grouped group_on_the_cpu(const Routed& r, size_t n_expert) {  // moe.rs:229-271 then :298-309, line by line
    std::vector<std::vector<std::pair<size_t, float>>> groups(n_expert);
    for (size_t i = 0; i < r.rows; i++)
        for (size_t j = 0; j < r.k; j++) groups[r.ids[i * r.k + j]].push_back({i, r.w[i * r.k + j]});
    Grouped g;
    uint32_t row0 = 0;
    std::vector<size_t> used;
    for (size_t e = 0; e < n_expert; e++)
        if (!groups[e].empty()) used.push_back(e);
    for (size_t e : used) {
        g.groups.push_back({(uint32_t)e, row0, (uint32_t)groups[e].size()});
        for (auto& p : groups[e]) g.tok.push_back((uint32_t)p.first);
        row0 += (uint32_t)groups[e].size();
    }
    g.total_rows = row0;
    std::vector<size_t> counts(r.rows, 0);
    g.hit_row.assign(r.rows * r.k, 0);
    g.hit_w.assign(r.rows * r.k, 0.0f);
    for (size_t gi = 0; gi < used.size(); gi++)
        for (size_t idx = 0; idx < groups[used[gi]].size(); idx++) {
            const size_t i = groups[used[gi]][idx].first;
            g.hit_row[i * r.k + counts[i]] = g.groups[gi][1] + (uint32_t)idx;
            g.hit_w[i * r.k + counts[i]] = groups[used[gi]][idx].second;
            counts[i]++;
        }
    g.tok_off.assign(r.rows + 1, 0);
    for (size_t i = 0; i < r.rows; i++) g.tok_off[i + 1] = g.tok_off[i] + (uint32_t)counts[i];
    return g;
}
static bool same_grouping(const Grouped& a, const Grouped& b) {
    return a.groups == b.groups && a.tok == b.tok && a.tok_off == b.tok_off && a.hit_row == b.hit_row && a.hit_w == b.hit_w &&
           a.total_rows == b.total_rows;
}
static void moe_group_orders_rows_by_expert_then_token() {  // moe.rs:229-271
    // 4 tokens, 2 picks each, 4 experts; expert 1 is never picked and gets no group
    Routed r = picks(4, 2, {2, 0, 0, 3, 2, 3, 0, 2}, {0.6f, 0.4f, 0.7f, 0.3f, 0.5f, 0.5f, 0.9f, 0.1f});
    Grouped g = moe_group(r, 4);
    CHECK((g.groups == std::vector<std::array<uint32_t, 3>>{{0, 0, 3}, {2, 3, 3}, {3, 6, 2}}));
    CHECK((g.tok == std::vector<uint32_t>{0, 1, 3, 0, 2, 3, 1, 2}));
    CHECK((g.tok_off == std::vector<uint32_t>{0, 2, 4, 6, 8}));
    CHECK((g.hit_row == std::vector<uint32_t>{0, 3, 1, 6, 4, 7, 2, 5}));
    CHECK((g.hit_w == std::vector<float>{0.4f, 0.6f, 0.7f, 0.3f, 0.5f, 0.5f, 0.9f, 0.1f}));
    CHECK(g.total_rows == 8);
    CHECK(same_grouping(g, group_on_the_cpu(r, 4)));
    // a larger batch with an uneven spread, picks straight from the device router
    const size_t rows = 300, n_expert = 24, k = 5;
    std::vector<float> logits(rows * n_expert);
    for (size_t i = 0; i < logits.size(); i++) logits[i] = std::sin(0.37f * (float)i) * 3.0f + ((i % n_expert) == 7 ? -40.0f : 0.0f);
    Routed rr = route_rows(logits, n_expert, k, Gating::Softmax, true, 1.0f, nullptr);
    CHECK(rr.rows == rows && rr.k == k);
    Grouped gg = moe_group(rr, n_expert);
    CHECK(same_grouping(gg, group_on_the_cpu(rr, n_expert)));
    for (auto& grp : gg.groups) CHECK(grp[0] != 7);  // nobody picks expert 7
    CHECK(throws<Panic>([] { moe_group(picks(1, 1, {9}, {1.0f}), 4); }));  // groups[9] of 4
    CHECK(moe_group(picks(0, 2, {}, {}), 4).total_rows == 0);
}
static void gather_then_combine_is_the_weighted_sum_of_the_hits() {  // moe.rs:298-333, :348-352
    const size_t rows = 50, n_expert = 8, k = 3, hidden = 256;
    std::vector<float> logits(rows * n_expert), x(rows * hidden), gamma(hidden);
    for (size_t i = 0; i < logits.size(); i++) logits[i] = std::cos(0.91f * (float)i);
    for (size_t i = 0; i < x.size(); i++) x[i] = std::sin(0.013f * (float)i) - 0.2f;
    for (size_t i = 0; i < hidden; i++) gamma[i] = 1.0f + 0.002f * (float)i;
    Routed r = route_rows(logits, n_expert, k, Gating::Softmax, true, 1.0f, nullptr);
    Grouped g = moe_group(r, n_expert);
    std::vector<float> xe = gather_rows(x, hidden, g, k);
    CHECK(xe.size() == g.total_rows * hidden);
    for (size_t row = 0; row < g.total_rows; row++)
        for (size_t i = 0; i < hidden; i += 17) CHECK(xe[row * hidden + i] == x[g.tok[row] * hidden + i]);
    // stand-in for the experts' down rows: twice the gathered row
    std::vector<float> flat(xe);
    for (float& v : flat) v *= 2.0f;
    std::vector<float> want(x), h(x.size(), 0.0f), got(x);
    for (size_t t = 0; t < rows; t++)
        for (size_t i = 0; i < hidden; i++) {
            float out = 0.0f;
            for (uint32_t j = g.tok_off[t]; j < g.tok_off[t + 1]; j++) out = std::fmaf(flat[g.hit_row[j] * hidden + i], g.hit_w[j], out);
            want[t * hidden + i] += out;
        }
    moe_combine_add_rmsnorm(got, flat, hidden, g, &h, &gamma, 1e-6f);
    for (size_t i = 0; i < got.size(); i++) CHECK(got[i] == want[i]);  // the same fused multiply-adds in the same order
    for (size_t t = 0; t < rows; t += 7) {
        double ss = 0.0;
        for (size_t i = 0; i < hidden; i++) ss += (double)want[t * hidden + i] * want[t * hidden + i];
        const double scale = 1.0 / std::sqrt(ss / hidden + 1e-6);
        for (size_t i = 0; i < hidden; i++) CHECK(close(h[t * hidden + i], (float)(want[t * hidden + i] * scale) * gamma[i]));
    }
    std::vector<float> plain(x);
    moe_combine_add_rmsnorm(plain, flat, hidden, g, nullptr, nullptr, 0.0f);  // the last layer: no next norm
    CHECK(plain == want);
    CHECK(throws<Panic>([&] { std::vector<float> shorter(flat.begin(), flat.end() - 1), xx(x); moe_combine_add_rmsnorm(xx, shorter, hidden, g, nullptr, nullptr, 0.0f); }));
}
static void argmax_is_the_last_maximum() {  // decode.rs:628-630: max_by(total_cmp)
    CHECK(argmax({0.5f, 3.0f, -1.0f, 2.0f}) == 1);
    CHECK(argmax({1.0f, 7.0f, 7.0f, 0.0f, 7.0f, 6.0f}) == 4);   // max_by keeps the last of equal maxima
    CHECK(argmax({0.0f, -0.0f}) == 0 && argmax({-0.0f, 0.0f}) == 1);  // total_cmp: -0.0 < +0.0
    CHECK(argmax({}) == 0);
    std::vector<float> wide(151936);
    for (size_t i = 0; i < wide.size(); i++) wide[i] = std::sin(0.001f * (float)i);
    size_t best = 0;
    for (size_t i = 0; i < wide.size(); i++)
        if (wide[i] >= wide[best]) best = i;
    CHECK(argmax(wide) == best);
}
static uint16_t half_bits(float f) {  // f16::from_f32, round to nearest even (values here are normal halves or zero)
    uint32_t u;
    std::memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int32_t exp = (int32_t)((u >> 23) & 0xff) - 127 + 15;
    uint32_t man = u & 0x7fffffu;
    if (exp <= 0) return (uint16_t)sign;  // flushed in this helper: the test keeps values well above 6e-5
    uint32_t h = ((uint32_t)exp << 10) | (man >> 13);
    const uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}
static void chunk_prologue_stores_the_rotated_k_and_v_rows() {  // attention.rs:131-200, kv.rs:682-697
    const size_t rows = 5, n_q = 4, n_kv = 2, hd = 128, capacity = 16;
    std::vector<float> q(rows * n_q * hd), k(rows * n_kv * hd), v(k.size()), qw(hd), kw(hd), inv(hd / 2);
    for (size_t i = 0; i < q.size(); i++) q[i] = 0.5f + std::sin(0.05f * (float)i);
    for (size_t i = 0; i < k.size(); i++) { k[i] = 0.5f + std::cos(0.03f * (float)i); v[i] = 1.0f + 0.25f * std::sin(0.11f * (float)i); }
    for (size_t i = 0; i < hd; i++) { qw[i] = 1.0f + 0.001f * (float)i; kw[i] = 1.0f - 0.001f * (float)i; }
    for (size_t i = 0; i < hd / 2; i++) inv[i] = std::pow(1e6f, -2.0f * (float)i / (float)hd);
    std::vector<uint32_t> pos = {3, 4, 5, 6, 9};
    auto rope = ops::rope_sin_cos_rows(pos, inv);
    std::vector<float> q2(q), k2(k);
    ops::qknorm_rope_rows(q2, k2, &qw, &kw, rope, rows, n_q, n_kv, hd, 1e-6f);
    KvLayer cache(capacity, n_kv * hd);
    cache.qknorm_rope_store(q, k, v, &qw, &kw, rope, pos, n_q, n_kv, hd, 1e-6f);
    CHECK(q == q2 && k == k2);  // the same arithmetic as the op without the store
    for (size_t r = 0; r < rows; r++) {
        auto kr = cache.k_row(pos[r]), vr = cache.v_row(pos[r]);
        for (size_t i = 0; i < n_kv * hd; i++) {
            CHECK(kr[i] == half_bits(k[r * n_kv * hd + i]));
            CHECK(vr[i] == half_bits(v[r * n_kv * hd + i]));
        }
    }
    CHECK(throws<Panic>([&] { std::vector<uint32_t> far = {1, 2, 3, 4, 16}; cache.qknorm_rope_store(q, k, v, &qw, &kw, rope, far, n_q, n_kv, hd, 1e-6f); }));
    CHECK(throws<Panic>([&] { std::vector<float> shortv(v.begin(), v.end() - 1); cache.qknorm_rope_store(q, k, shortv, &qw, &kw, rope, pos, n_q, n_kv, hd, 1e-6f); }));
}

int main() {
    struct { const char* name; void (*fn)(); } tests[] = {
        {"rmsnorm_normalises_to_unit_rms_before_the_weight", rmsnorm_normalises_to_unit_rms_before_the_weight},
        {"rmsnorm_applies_the_weight_per_channel", rmsnorm_applies_the_weight_per_channel},
        {"rmsnorm_eps_keeps_zero_input_finite", rmsnorm_eps_keeps_zero_input_finite},
        {"rmsnorm_rows_into_rejects_a_short_destination", rmsnorm_rows_into_rejects_a_short_destination},
        {"add_assign_then_norm_matches_the_two_ops", add_assign_then_norm_matches_the_two_ops},
        {"sandwich_norm_matches_the_three_ops", sandwich_norm_matches_the_three_ops},
        {"add_bias_rows_biases_every_whole_row", add_bias_rows_biases_every_whole_row},
        {"swiglu_is_silu_of_gate_times_up", swiglu_is_silu_of_gate_times_up},
        {"geglu_tanh_is_the_tanh_gelu_of_gate_times_up", geglu_tanh_is_the_tanh_gelu_of_gate_times_up},
        {"softmax_sums_to_one_and_survives_huge_logits", softmax_sums_to_one_and_survives_huge_logits},
        {"add_assign_slice_adds_and_rejects_length_mismatch", add_assign_slice_adds_and_rejects_length_mismatch},
        {"add_scaled_slice_is_one_fma_and_rejects_length_mismatch", add_scaled_slice_is_one_fma_and_rejects_length_mismatch},
        {"rope_is_norm_preserving_and_identity_at_position_zero", rope_is_norm_preserving_and_identity_at_position_zero},
        {"rope_neox_pairs_split_channels", rope_neox_pairs_split_channels},
        {"partial_rotary_rotates_the_head_and_passes_the_tail", partial_rotary_rotates_the_head_and_passes_the_tail},
        {"device_rope_rows_match_the_host_table", device_rope_rows_match_the_host_table},
        {"q8_0_is_scale_times_value", q8_0_is_scale_times_value},
        {"weights_are_named_by_host_address_inside_an_attached_mapping", weights_are_named_by_host_address_inside_an_attached_mapping},
        {"route_picks_the_top_k_and_renormalises", route_picks_the_top_k_and_renormalises},
        {"moe_group_orders_rows_by_expert_then_token", moe_group_orders_rows_by_expert_then_token},
        {"gather_then_combine_is_the_weighted_sum_of_the_hits", gather_then_combine_is_the_weighted_sum_of_the_hits},
        {"argmax_is_the_last_maximum", argmax_is_the_last_maximum},
        {"chunk_prologue_stores_the_rotated_k_and_v_rows", chunk_prologue_stores_the_rotated_k_and_v_rows},
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

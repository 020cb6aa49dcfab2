// host_mirror_test.cpp -- the C++ host layer (include/dsx_moe.hpp) exercised the way the
// reference's own rigs exercise its Rust wrappers (crates/v4flash-kernels/tests/
// mtp_moe_grouped.rs:129-176, mxfp4_pair_oracle.rs:86-100,176): operators one by one through
// the wrappers, then the executor, each result against the CPU oracle on the same seeded input.
//
//   host_mirror_test --host-only   checks that need no GPU: argument refusals before any launch,
//                                  views, the work-item bound's known answers
//   host_mirror_test               the above plus the GPU parity cases
//
// Test infrastructure: links the oracle; nothing here is part of the shipped library.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "dsx_moe.hpp"
#include "dsx_oracle.h"

namespace {

int g_checks = 0, g_failed = 0;

void expect(bool cond, const char *what, const std::string &detail = "") {
    g_checks++;
    if (!cond) {
        g_failed++;
        std::printf("FAIL %s %s\n", what, detail.c_str());
    } else {
        std::printf("ok   %s %s\n", what, detail.c_str());
    }
    std::fflush(stdout);
}

bool must(const dsx::Status &st, const char *what) {
    if (st.ok()) return true;
    g_checks++;
    g_failed++;
    std::printf("FAIL %s: status %d: %s\n", what, st.code, st.message.c_str());
    std::fflush(stdout);
    return false;
}

// max |a - b| / max |ref|  (crates/v4flash-kernels/tests/mxfp4_pair_oracle.rs:86-100)
double rel_err(const std::vector<float> &a, const float *ref, size_t n) {
    double mx = 0.0, d = 0.0;
    for (size_t i = 0; i < n; i++) {
        mx = std::max(mx, (double)std::fabs(ref[i]));
        d = std::max(d, (double)std::fabs(a[i] - ref[i]));
    }
    return mx > 0.0 ? d / mx : d;
}

std::string sci(double v) {
    char buf[32];
    std::snprintf(buf, sizeof buf, "%.2e", v);
    return buf;
}

std::vector<float> normals(std::mt19937_64 &rng, size_t n, float sigma) {
    std::normal_distribution<float> dist(0.0f, sigma);
    std::vector<float> v(n);
    for (auto &x : v) x = dist(rng);
    return v;
}

// ---- checks without a GPU ---------------------------------------------------------------------
void host_only_checks() {
    using namespace dsx;
    // crates/v4flash-kernels/src/het/dispatch.rs:721-749 (the reference's known answers)
    expect(dispatch::moe_wi_upper_bound(12, 384, 32, 1u << 20) == 12, "moe_wi_upper_bound(12,384,32)");
    expect(dispatch::moe_wi_upper_bound(3072, 384, 32, 1u << 20) == 480, "moe_wi_upper_bound(3072,384,32)");
    expect(dispatch::moe_wi_upper_bound(3072, 384, 32, 100) == 100, "moe_wi_upper_bound capped");
    for (size_t m : {0u, 1u, 7u, 48u, 1000u})
        for (uint32_t g : {1u, 16u, 256u})
            for (uint32_t c : {1u, 4u, 32u})
                if (dispatch::moe_wi_upper_bound(m, g, c, 1u << 20) != dsx_ref_wi_upper_bound(m, g, c, 1u << 20))
                    expect(false, "moe_wi_upper_bound vs oracle");

    expect(act_row_bytes(GgufType::MXFP4, 7168) == 8176, "Q8_K row of 7168 is 8176 bytes");
    expect(act_row_bytes(GgufType::Q8_0, 1408) == 1408 + 176, "Q8_0 activation row of 1408");
    expect(weight_row_bytes(GgufType::MXFP4, 2048) * 7168 == 7798784, "MXFP4 7168x2048 matrix is 7,798,784 bytes");
    expect(weight_row_bytes(GgufType::Q8_0, 2048) * 7168 == 15597568, "Q8_0 7168x2048 matrix is 15,597,568 bytes");

    // views: a slice_view never reaches past its parent
    float *fake = reinterpret_cast<float *>(0x1000);  // never dereferenced: every call below is refused first
    DeviceSlice<float> whole(fake, 100);
    expect(whole.slice_view(10, 90).len() == 90 && whole.slice_view(10, 90).ptr() == fake + 10, "slice_view in range");
    expect(whole.slice_view(10, 91).empty() && whole.slice_view(101, 0).empty(), "slice_view out of range is empty");

    // refusals before any launch, with the reference's "have / need" wording
    // (crates/v4flash-kernels/src/q8_k.rs:40-55)
    Stream s = Stream::borrowed(nullptr);
    uint8_t *fake8 = reinterpret_cast<uint8_t *>(0x2000);
    Status st = Q8KQuantize::launch(s, Out<uint8_t>(fake8, 292 * 4), In<float>(fake, 256 * 3), 4);
    expect(!st.ok() && st.code == DSX_ERR_INVALID_ARG && st.message.find("have 768, need 1024") != std::string::npos,
           "Q8KQuantize refuses a short x", st.message);
    st = Q8KQuantize::launch(s, Out<uint8_t>(fake8, 292 * 3), In<float>(fake, 256 * 4), 4);
    expect(!st.ok() && st.message.find("out bytes") != std::string::npos, "Q8KQuantize refuses a short out", st.message);
    int32_t *fakei = reinterpret_cast<int32_t *>(0x3000);
    st = RouterTopk::launch_batched_ex(s, Out<int32_t>(fakei, 8), Out<float>(fake, 8), In<float>(fake, 63), {}, 64, 8,
                                       1.5f, 6.1e-5f, 1, RouterMode::SqrtSoftplus);
    expect(!st.ok() && st.code == DSX_ERR_INVALID_ARG, "RouterTopk refuses short logits", st.message);
    st = dispatch::moe_gate_up_batch(GgufType::MXFP4, s, Out<float>(fake, 8 * 2048), In<uint8_t>(fake8, 7798784),
                                     In<uint8_t>(fake8, 7798784), In<uint8_t>(fake8, 8176), In<float>(fake, 8),
                                     In<int32_t>(fakei, 8), 7798784 - 136, 7798784, 8, 10.0f, 2048, 28);
    expect(!st.ok() && st.code == DSX_ERR_SHAPE, "moe_gate_up_batch refuses bytes-per-expert below n_rows rows",
           st.message);
    st = dispatch::reduce_partials(s, Out<float>(fake, 100), In<float>(fake, 100), {}, 8, 64, 2);
    expect(!st.ok(), "reduce_partials refuses a short out", st.message);
    st = HcPost::launch_batched(s, Out<float>(fake, 2 * 4 * 64), In<float>(fake, 2 * 64), In<float>(fake, 2 * 4 * 64),
                                In<float>(fake, 8), In<float>(fake, 31), 64, 4, 2);
    expect(!st.ok() && st.message.find("hc_post comb") != std::string::npos, "HcPost refuses a short comb", st.message);
    MoeExecutor none;
    st = none.run(s, Out<float>(fake, 16), In<float>(fake, 16), In<float>(fake, 16), 1);
    expect(!st.ok() && st.message.find("not created") != std::string::npos, "MoeExecutor refuses to run uncreated");
    st = for_arch("gfx1151");
    expect(!st.ok() && st.code == DSX_ERR_DEVICE, "for_arch refuses another architecture", st.message);
    // what the C entry points themselves refuse (a second line of defence under the wrappers)
    expect(dsx_q8k_quantize(nullptr, nullptr, fake, 4) == DSX_ERR_INVALID_ARG, "C ABI refuses a null out");
    expect(dsx_abi_version() == DSX_ABI_VERSION, "ABI version");
}

// ---- synthetic layer --------------------------------------------------------------------------
struct HostLayer {
    int hidden, inter, n_expert, n_used, sh_inter;
    dsx::GgufType fmt;
    std::vector<uint8_t> gate, up, down, sh_gate, sh_up, sh_down;
    uint64_t gate_bpe, down_bpe;
};

std::vector<uint8_t> quantize(dsx::GgufType fmt, const std::vector<float> &w, size_t rows, size_t cols) {
    std::vector<uint8_t> out(rows * dsx::weight_row_bytes(fmt, (uint32_t)cols));
    if (fmt == dsx::GgufType::MXFP4) dsx_ref_mxfp4_quantize_v2(w.data(), out.data(), rows, cols);
    else dsx_ref_q8_0_quantize_rows(w.data(), out.data(), rows, cols);
    return out;
}

HostLayer make_layer(std::mt19937_64 &rng, dsx::GgufType fmt, int hidden, int inter, int n_expert, int n_used,
                     int sh_inter) {
    HostLayer L{hidden, inter, n_expert, n_used, sh_inter, fmt, {}, {}, {}, {}, {}, {}, 0, 0};
    const float sigma = 0.05f;
    L.gate = quantize(fmt, normals(rng, (size_t)n_expert * inter * hidden, sigma), (size_t)n_expert * inter, hidden);
    L.up = quantize(fmt, normals(rng, (size_t)n_expert * inter * hidden, sigma), (size_t)n_expert * inter, hidden);
    L.down = quantize(fmt, normals(rng, (size_t)n_expert * hidden * inter, sigma), (size_t)n_expert * hidden, inter);
    L.gate_bpe = (uint64_t)inter * dsx::weight_row_bytes(fmt, hidden);
    L.down_bpe = (uint64_t)hidden * dsx::weight_row_bytes(fmt, inter);
    if (sh_inter > 0) {
        L.sh_gate = quantize(fmt, normals(rng, (size_t)sh_inter * hidden, sigma), sh_inter, hidden);
        L.sh_up = quantize(fmt, normals(rng, (size_t)sh_inter * hidden, sigma), sh_inter, hidden);
        L.sh_down = quantize(fmt, normals(rng, (size_t)hidden * sh_inter, sigma), hidden, sh_inter);
    }
    return L;
}

dsx_ref_moe_cfg ref_cfg(const HostLayer &L, bool with_shared) {
    dsx_ref_moe_cfg c{};
    c.hidden = L.hidden; c.inter = L.inter; c.n_expert = L.n_expert; c.n_used = L.n_used;
    c.gate_fmt = c.up_fmt = c.down_fmt = (int)L.fmt;
    c.gate = L.gate.data(); c.up = L.up.data(); c.down = L.down.data();
    c.gate_bpe = c.up_bpe = L.gate_bpe; c.down_bpe = L.down_bpe;
    c.clamp = 10.0f;
    if (with_shared && L.sh_inter > 0) {
        c.sh_inter = L.sh_inter;
        c.sh_gate_fmt = c.sh_up_fmt = c.sh_down_fmt = (int)L.fmt;
        c.sh_gate = L.sh_gate.data(); c.sh_up = L.sh_up.data(); c.sh_down = L.sh_down.data();
        c.sh_clamp = 10.0f;
    }
    return c;
}

// picks must match exactly wherever the gap between the k-th and (k+1)-th score exceeds 1e-4
bool picks_agree(const std::vector<int32_t> &got, const std::vector<int32_t> &want, const std::vector<float> &scores,
                 int T, int E, int k) {
    for (int t = 0; t < T; t++) {
        if (std::equal(got.begin() + t * k, got.begin() + (t + 1) * k, want.begin() + t * k)) continue;
        std::vector<float> s(scores.begin() + (size_t)t * E, scores.begin() + (size_t)(t + 1) * E);
        std::sort(s.begin(), s.end(), std::greater<float>());
        bool near_tie = false;
        for (int i = 0; i + 1 < E && i < k + 1; i++) near_tie |= (s[i] - s[i + 1]) <= 1e-4f;
        if (!near_tie) return false;
    }
    return true;
}

struct RouterCfg { dsx::RouterMode mode; bool bias; uint32_t n_group, topk_group; float scale, eps; };

// ---- one layer shape through every wrapper -----------------------------------------------------
void gpu_case(const char *name, dsx::GgufType fmt, int hidden, int inter, int E, int k, int sh_inter, int T,
              RouterCfg rc, uint64_t seed) {
    using namespace dsx;
    std::printf("== %s: fmt %d hidden %d inter %d experts %d top-%d shared %d T %d seed %llu\n", name, (int)fmt, hidden,
                inter, E, k, sh_inter, T, (unsigned long long)seed);
    std::fflush(stdout);
    std::mt19937_64 rng(seed);
    HostLayer L = make_layer(rng, fmt, hidden, inter, E, k, sh_inter);
    std::vector<float> x = normals(rng, (size_t)T * hidden, 1.0f);
    std::vector<float> logits = normals(rng, (size_t)T * E, 1.0f);
    std::vector<float> bias = rc.bias ? normals(rng, E, 0.01f) : std::vector<float>();

    // oracle
    std::vector<int32_t> sel_ref((size_t)T * k);
    std::vector<float> w_ref((size_t)T * k), probs((size_t)T * E), scores((size_t)T * E);
    const float *bias_p = rc.bias ? bias.data() : nullptr;
    dsx_ref_router_topk(sel_ref.data(), w_ref.data(), logits.data(), bias_p, E, k, rc.scale, rc.eps, T, (int)rc.mode,
                        (int)rc.n_group, (int)rc.topk_group);
    dsx_ref_router_scores(probs.data(), scores.data(), logits.data(), bias_p, E, T, (int)rc.mode, (int)rc.n_group,
                          (int)rc.topk_group);
    dsx_ref_moe_cfg c_routed = ref_cfg(L, false), c_full = ref_cfg(L, true);
    std::vector<float> out_routed((size_t)T * hidden), out_full((size_t)T * hidden), mid_ref((size_t)T * k * inter);
    dsx_ref_moe_forward(&c_routed, x.data(), sel_ref.data(), w_ref.data(), T, out_routed.data(), mid_ref.data(),
                        nullptr, nullptr, 0);
    dsx_ref_moe_forward(&c_full, x.data(), sel_ref.data(), w_ref.data(), T, out_full.data(), nullptr, nullptr,
                        nullptr, 0);

    // device
    Stream s;
    if (!must(Stream::create(s), "Stream::create")) return;
    DeviceBuffer<uint8_t> d_gate, d_up, d_down, d_shg, d_shu, d_shd;
    DeviceBuffer<float> d_x, d_logits, d_bias;
    if (!must(DeviceBuffer<uint8_t>::from_host(d_gate, L.gate), "gate") ||
        !must(DeviceBuffer<uint8_t>::from_host(d_up, L.up), "up") ||
        !must(DeviceBuffer<uint8_t>::from_host(d_down, L.down), "down") ||
        !must(DeviceBuffer<uint8_t>::from_host(d_shg, L.sh_gate), "sh_gate") ||
        !must(DeviceBuffer<uint8_t>::from_host(d_shu, L.sh_up), "sh_up") ||
        !must(DeviceBuffer<uint8_t>::from_host(d_shd, L.sh_down), "sh_down") ||
        !must(DeviceBuffer<float>::from_host(d_x, x), "x") ||
        !must(DeviceBuffer<float>::from_host(d_logits, logits), "logits") ||
        !must(DeviceBuffer<float>::from_host(d_bias, bias), "bias"))
        return;

    // 1. router
    DeviceBuffer<int32_t> d_sel;
    DeviceBuffer<float> d_w;
    if (!must(DeviceBuffer<int32_t>::zeroed(d_sel, (size_t)T * k), "sel") ||
        !must(DeviceBuffer<float>::zeroed(d_w, (size_t)T * k), "w"))
        return;
    if (!must(RouterTopk::launch_batched_ex(s, d_sel, d_w, d_logits, d_bias, E, k, rc.scale, rc.eps, T, rc.mode,
                                            rc.n_group, rc.topk_group),
              "RouterTopk::launch_batched_ex"))
        return;
    if (!must(s.synchronize(), "sync")) return;
    std::vector<int32_t> sel;
    std::vector<float> w;
    if (!must(d_sel.copy_to_host(sel), "sel back") || !must(d_w.copy_to_host(w), "w back")) return;
    expect(picks_agree(sel, sel_ref, scores, T, E, k), "router picks equal the oracle's (gap > 1e-4)");
    const bool same_picks = sel == sel_ref;
    if (same_picks) expect(rel_err(w, w_ref.data(), w.size()) < 1e-5, "router weights");
    // everything below runs on the oracle's picks so that a near tie cannot leak into the products
    if (!must(d_sel.copy_from_host(sel_ref.data(), sel_ref.size()), "sel ref") ||
        !must(d_w.copy_from_host(w_ref.data(), w_ref.size()), "w ref"))
        return;

    const uint32_t nb_in = fmt == GgufType::MXFP4 ? hidden / 256 : hidden / 32;
    const uint32_t nb_mid = fmt == GgufType::MXFP4 ? inter / 256 : inter / 32;
    const uint32_t x_row = (uint32_t)act_row_bytes(fmt, hidden), mid_row = (uint32_t)act_row_bytes(fmt, inter);

    // 2. by-expert operators: quantize -> group build -> gate/up -> quantize -> down -> reduce
    //    (crates/v4flash-kernels/tests/mtp_moe_grouped.rs:129-176)
    {
        const uint32_t chunk = 4;
        DeviceBuffer<uint8_t> d_xq, d_midq;
        DeviceBuffer<float> d_mid, d_partials, d_out;
        MoeGroups groups;
        if (!must(DeviceBuffer<uint8_t>::zeroed(d_xq, (size_t)T * x_row), "xq") ||
            !must(DeviceBuffer<uint8_t>::zeroed(d_midq, (size_t)T * k * mid_row), "midq") ||
            !must(DeviceBuffer<float>::zeroed(d_mid, (size_t)T * k * inter), "mid") ||
            !must(DeviceBuffer<float>::zeroed(d_partials, (size_t)T * k * hidden), "partials") ||
            !must(DeviceBuffer<float>::zeroed(d_out, (size_t)T * hidden), "out") ||
            !must(MoeGroups::alloc(groups, E, (uint32_t)T * k), "groups"))
            return;
        const uint32_t max_wi = dispatch::moe_wi_upper_bound((size_t)T * k, E, chunk, groups.work_items.len());
        bool ok = must(quantize_rows(s, fmt, d_xq, d_x, T, hidden), "quantize_rows x") &&
                  must(MoeGroupBuilder::launch(s, groups, d_sel, T, k, E, chunk), "MoeGroupBuilder::launch") &&
                  must(dispatch::moe_gate_up_chunked_rows(fmt, s, d_mid, d_gate, d_up, d_xq, d_w, groups, max_wi,
                                                          L.gate_bpe, L.gate_bpe, k, chunk, 10.0f, inter, nb_in, T),
                       "moe_gate_up_chunked_rows") &&
                  must(quantize_rows(s, fmt, d_midq, d_mid, (uint32_t)T * k, inter), "quantize_rows mid") &&
                  must(dispatch::moe_down_mxfp4(fmt, s, d_partials, d_down, d_midq, groups, max_wi, L.down_bpe,
                                                mid_row, k, chunk, hidden, nb_mid, T),
                       "moe_down_mxfp4") &&
                  must(dispatch::reduce_partials(s, d_out, d_partials, d_sel, k, hidden, T), "reduce_partials") &&
                  must(s.synchronize(), "sync");
        if (!ok) return;
        std::vector<float> mid, out;
        std::vector<int32_t> n_wi, cnt;
        if (!must(d_mid.copy_to_host(mid), "mid back") || !must(d_out.copy_to_host(out), "out back") ||
            !must(groups.n_work_items.copy_to_host(n_wi), "n_wi back") ||
            !must(groups.group_count.copy_to_host(cnt), "count back"))
            return;
        std::vector<int32_t> r_cnt(E), r_off(E + 1), r_mem((size_t)T * k), r_wi((size_t)T * k + E);
        const int r_n = dsx_ref_group_build(r_cnt.data(), r_off.data(), r_mem.data(), r_wi.data(), sel_ref.data(), T, k,
                                            E, (int)chunk);
        expect(n_wi[0] == r_n && cnt == r_cnt && (uint32_t)r_n <= max_wi, "group tables equal the oracle's",
               "work items " + std::to_string(n_wi[0]) + " (bound " + std::to_string(max_wi) + ")");
        const double e_mid = rel_err(mid, mid_ref.data(), mid.size());
        const double e_out = rel_err(out, out_routed.data(), out.size());
        expect(e_mid < 2e-3, "by-expert gate/up + SwiGLU", "rel " + sci(e_mid));
        expect(e_out < 2e-3, "by-expert down + slot-order reduce", "rel " + sci(e_out));
    }

    // 3. decode operators on token 0 (crates/v4flash-kernels/src/het/forward_layer.rs:456-466)
    {
        DeviceBuffer<uint8_t> d_xq, d_midq;
        DeviceBuffer<float> d_mid, d_out;
        if (!must(DeviceBuffer<uint8_t>::zeroed(d_xq, x_row), "xq") ||
            !must(DeviceBuffer<uint8_t>::zeroed(d_midq, (size_t)k * mid_row), "midq") ||
            !must(DeviceBuffer<float>::zeroed(d_mid, (size_t)k * inter), "mid") ||
            !must(DeviceBuffer<float>::zeroed(d_out, hidden), "out"))
            return;
        bool ok = must(quantize_rows(s, fmt, d_xq, d_x.slice_view(0, hidden), 1, hidden), "quantize_rows x[0]") &&
                  must(dispatch::moe_gate_up_batch(fmt, s, d_mid, d_gate, d_up, d_xq, d_w.slice_view(0, k),
                                                   d_sel.slice_view(0, k), L.gate_bpe, L.gate_bpe, k, 10.0f, inter,
                                                   nb_in),
                       "moe_gate_up_batch") &&
                  must(quantize_rows(s, fmt, d_midq, d_mid, k, inter), "quantize_rows mid") &&
                  must(dispatch::moe_down_batched(fmt, s, d_out, d_down, d_midq, d_sel.slice_view(0, k), L.down_bpe,
                                                  mid_row, k, hidden, nb_mid),
                       "moe_down_batched") &&
                  must(s.synchronize(), "sync");
        if (!ok) return;
        std::vector<float> out;
        if (!must(d_out.copy_to_host(out), "out back")) return;
        const double e = rel_err(out, out_routed.data(), hidden);
        expect(e < 2e-3, "decode operators, token 0", "rel " + sci(e));
    }

    // 4. executor: router + routed experts + shared expert in one call
    {
        dsx_moe_layer_desc d{};
        d.hidden = hidden; d.inter = inter; d.n_expert = E; d.n_used = k;
        d.gate_fmt = d.up_fmt = d.down_fmt = (int)fmt;
        d.gate = d_gate.ptr(); d.up = d_up.ptr(); d.down = d_down.ptr();
        d.gate_bpe = d.up_bpe = L.gate_bpe; d.down_bpe = L.down_bpe;
        d.clamp = 10.0f;
        d.router_mode = (uint32_t)rc.mode; d.n_group = rc.n_group; d.topk_group = rc.topk_group;
        d.route_scale = rc.scale; d.route_eps = rc.eps;
        d.bias = rc.bias ? d_bias.ptr() : nullptr;
        if (sh_inter > 0) {
            d.sh_inter = sh_inter;
            d.sh_gate_fmt = d.sh_up_fmt = d.sh_down_fmt = (int)fmt;
            d.sh_gate = d_shg.ptr(); d.sh_up = d_shu.ptr(); d.sh_down = d_shd.ptr();
            d.sh_clamp = 10.0f;
        }
        MoeExecutor ex;
        DeviceBuffer<float> d_out;
        DeviceBuffer<int32_t> d_sel2;
        if (!must(MoeExecutor::create(ex, d, T), "MoeExecutor::create") ||
            !must(DeviceBuffer<float>::zeroed(d_out, (size_t)T * hidden), "out") ||
            !must(DeviceBuffer<int32_t>::zeroed(d_sel2, (size_t)T * k), "sel2"))
            return;
        Status st = ex.run(s, d_out, d_x, d_logits, T + 1);
        expect(!st.ok() && st.code == DSX_ERR_INVALID_ARG, "MoeExecutor refuses more tokens than it was sized for",
               st.message);
        st = ex.run(s, d_out.slice_view(0, (size_t)T * hidden - 1), d_x, d_logits, T);
        expect(!st.ok(), "MoeExecutor refuses a short out", st.message);
        std::vector<float> out;
        std::vector<int32_t> sel2;
        if (same_picks) {
            if (!must(ex.run(s, d_out, d_x, d_logits, T, d_sel2), "MoeExecutor::run") || !must(s.synchronize(), "sync") ||
                !must(d_out.copy_to_host(out), "out back") || !must(d_sel2.copy_to_host(sel2), "sel2 back"))
                return;
            const double e = rel_err(out, out_full.data(), out.size());
            expect(sel2 == sel_ref && e < 2e-3, "MoeExecutor::run (router inside)", "rel " + sci(e));
        }
        if (!must(ex.run_selected(s, d_out, d_x, d_sel, d_w, T), "MoeExecutor::run_selected") ||
            !must(s.synchronize(), "sync") || !must(d_out.copy_to_host(out), "out back"))
            return;
        const double e = rel_err(out, out_full.data(), out.size());
        expect(e < 2e-3, "MoeExecutor::run_selected (picks given)", "rel " + sci(e));
        // one token through the same executor: the decode path of the layer
        if (!must(ex.run_selected(s, d_out, d_x, d_sel, d_w, 1), "MoeExecutor::run_selected T=1") ||
            !must(s.synchronize(), "sync") || !must(d_out.copy_to_host(out), "out back"))
            return;
        const double e1 = rel_err(out, out_full.data(), hidden);
        expect(e1 < 2e-3, "MoeExecutor::run_selected, one token", "rel " + sci(e1));
    }
}

}  // namespace

// HcPost (crates/v4flash-kernels/src/head.rs:269-500) through the wrappers, bit for bit against the oracle:
// separate post / comb arrays, then the same values inside packed split rows with both addends.
void hc_post_case() {
    using namespace dsx;
    const uint32_t b = 3, n_hc = 4, n_embd = 512, n_w = 5, stride = n_w + n_hc + n_hc * n_hc;
    std::mt19937_64 rng(77);
    const auto block = normals(rng, (size_t)b * n_embd, 1.0f), a1 = normals(rng, (size_t)b * n_embd, 1.0f);
    const auto a2 = normals(rng, (size_t)b * n_embd, 1.0f), res = normals(rng, (size_t)b * n_hc * n_embd, 1.0f);
    const auto split = normals(rng, (size_t)b * stride, 1.0f);
    std::vector<float> post((size_t)b * n_hc), comb((size_t)b * n_hc * n_hc);
    for (uint32_t t = 0; t < b; t++) {
        std::copy_n(&split[(size_t)t * stride + n_w], n_hc, &post[(size_t)t * n_hc]);
        std::copy_n(&split[(size_t)t * stride + n_w + n_hc], n_hc * n_hc, &comb[(size_t)t * n_hc * n_hc]);
    }
    Stream s;
    if (!must(Stream::create(s), "hc_post stream")) return;
    DeviceBuffer<float> d_block, d_a1, d_a2, d_res, d_split, d_post, d_comb, d_out;
    if (!must(DeviceBuffer<float>::from_host(d_block, block), "hc_post upload") ||
        !must(DeviceBuffer<float>::from_host(d_a1, a1), "hc_post upload") ||
        !must(DeviceBuffer<float>::from_host(d_a2, a2), "hc_post upload") ||
        !must(DeviceBuffer<float>::from_host(d_res, res), "hc_post upload") ||
        !must(DeviceBuffer<float>::from_host(d_split, split), "hc_post upload") ||
        !must(DeviceBuffer<float>::from_host(d_post, post), "hc_post upload") ||
        !must(DeviceBuffer<float>::from_host(d_comb, comb), "hc_post upload") ||
        !must(DeviceBuffer<float>::zeroed(d_out, res.size()), "hc_post out"))
        return;
    std::vector<float> got(res.size()), want(res.size());
    if (!must(HcPost::launch_batched(s, d_out.view(), d_block.view(), d_res.view(), d_post.view(), d_comb.view(),
                                     n_embd, n_hc, b), "HcPost::launch_batched") ||
        !must(s.synchronize(), "hc_post sync") || !must(d_out.copy_to_host(got), "hc_post download"))
        return;
    dsx_ref_hc_post(want.data(), block.data(), nullptr, nullptr, res.data(), post.data(), comb.data(), n_embd, n_hc,
                    b, n_hc, n_hc * n_hc);
    expect(std::memcmp(got.data(), want.data(), got.size() * 4) == 0, "HcPost::launch_batched equals the oracle bit for bit");
    if (!must(HcPost::launch_from_split_batched_add2(s, d_out.view(), d_block.view(), d_a1.view(), d_a2.view(),
                                                     d_res.view(), d_split.view(), n_w, n_embd, n_hc, b),
              "HcPost::launch_from_split_batched_add2") ||
        !must(s.synchronize(), "hc_post sync") || !must(d_out.copy_to_host(got), "hc_post download"))
        return;
    dsx_ref_hc_post(want.data(), block.data(), a1.data(), a2.data(), res.data(), split.data() + n_w,
                    split.data() + n_w + n_hc, n_embd, n_hc, b, stride, stride);
    expect(std::memcmp(got.data(), want.data(), got.size() * 4) == 0,
           "HcPost::launch_from_split_batched_add2 equals the oracle bit for bit");
}

int main(int argc, char **argv) {
    const bool host_only = argc > 1 && std::strcmp(argv[1], "--host-only") == 0;
    host_only_checks();
    if (!host_only) {
        dsx::Status st = dsx::for_arch("gfx950");
        if (!must(st, "for_arch(gfx950)")) return 2;
        // the V3 router (sigmoid + bias, group-limited, scale 2.5) on MXFP4 with a shared expert
        gpu_case("mxfp4 sigmoid group-limited", dsx::GgufType::MXFP4, 512, 256, 16, 4, 256, 7,
                 {dsx::RouterMode::Sigmoid, true, 4, 2, 2.5f, 1e-20f}, 0xD5EE0001ull);
        // the engine's own router (sqrt-softplus, scale 1.5) on MXFP4, no shared expert
        gpu_case("mxfp4 sqrt-softplus", dsx::GgufType::MXFP4, 768, 512, 32, 6, 0, 5,
                 {dsx::RouterMode::SqrtSoftplus, false, 1, 1, 1.5f, 6.103515625e-5f}, 0xD5EE0002ull);
        // the CPU-runnable configuration's kind: Q8_0 everywhere, softmax top-6, inter a multiple of
        // 128 (what the Q8_0 rows need) but not of 256
        gpu_case("q8_0 softmax", dsx::GgufType::Q8_0, 256, 384, 16, 6, 384, 4,
                 {dsx::RouterMode::Softmax, false, 1, 1, 1.0f, 1e-20f}, 0xD5EE0003ull);
    }
    if (!host_only) hc_post_case();
    std::printf("%s: %d checks, %d failed%s\n", g_failed == 0 ? "PASS" : "FAIL", g_checks, g_failed,
                host_only ? " (host only)" : "");
    return g_failed == 0 ? 0 : 1;
}

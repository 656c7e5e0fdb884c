// Parity driver for HipQ8Backend: every op is called the way the reference's
// executor and its own backend tests call it (tests/mixed_linear_parity.cu:205-278
// for the closed-form case) and checked against the CPU oracle on seeded inputs.
// Prints one line per case; exit code 0 only if all pass.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <string>
#include <vector>

#include <unistd.h>

#include "../../kvmem-qw3_amd/host/hip_q8_backend.hpp"
#include "../../kvmem-qw3_amd/host/gguf_q8.hpp"
#include "../../oracle/q8_oracle.h"

namespace {

int g_failed = 0;
int g_cases = 0;

void report(const char *name, bool ok, const std::string &detail = "") {
    ++g_cases;
    if (!ok) ++g_failed;
    std::printf("%s %s%s%s\n", ok ? "PASS" : "FAIL", name, detail.empty() ? "" : ": ", detail.c_str());
    std::fflush(stdout);
}

bool require(const qw3::DeviceStatus &st, const char *what) {
    if (!st.ok) {
        std::printf("  status: %s: %s\n", what, st.message);
        std::fflush(stdout);
    }
    return st.ok;
}

struct Rng {   // splitmix64
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed) {}
    uint64_t next() {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    float uniform() { return static_cast<float>(next() >> 40) * (1.0f / 16777216.0f); }
    float normal() {
        const float u1 = uniform() + 1e-7f, u2 = uniform();
        return std::sqrt(-2.0f * std::log(u1)) * std::cos(6.2831853f * u2);
    }
};

std::vector<float> normal_vec(size_t n, uint64_t seed, float scale = 1.0f) {
    Rng r(seed);
    std::vector<float> v(n);
    for (auto &f : v) f = r.normal() * scale;
    return v;
}

struct HostWeight {
    uint32_t rows, cols;
    std::vector<uint8_t> gguf;    // interleaved blocks handed to weight_q8_0
    std::vector<uint8_t> split;   // oracle's split-plane copy
};

HostWeight make_weight(uint32_t rows, uint32_t cols, uint64_t seed) {
    HostWeight w{rows, cols, {}, {}};
    const auto vals = normal_vec(static_cast<size_t>(rows) * cols, seed, 0.05f);
    w.gguf.resize(static_cast<size_t>(rows) * (cols / 32) * 34);
    w.split.resize(w.gguf.size());
    q8o_quantize_q8_0(vals.data(), rows, cols, w.gguf.data());
    q8o_repack_split_plane(w.gguf.data(), rows, cols, w.split.data());
    return w;
}

// oracle result for any batch (slices of 8, like the reference's GEMV dispatch)
void oracle_linear(const HostWeight &w, const float *x, uint32_t batch, uint32_t in_stride, uint32_t out_stride,
                   std::vector<float> &ref, std::vector<float> &mag) {
    ref.assign(static_cast<size_t>(batch) * out_stride, 0.0f);
    mag.assign(ref.size(), 0.0f);
    std::vector<uint8_t> y(static_cast<size_t>(8) * (w.cols / 32) * 36);
    for (uint32_t j0 = 0; j0 < batch; j0 += 8) {
        const uint32_t m = batch - j0 < 8 ? batch - j0 : 8;
        q8o_quantize_q8_1(x + static_cast<size_t>(j0) * in_stride, m, w.cols, in_stride, y.data());
        q8o_gemv(w.split.data(), y.data(), ref.data() + static_cast<size_t>(j0) * out_stride, w.rows, w.cols, m,
                 out_stride, 4);
        q8o_gemv_abs(w.split.data(), y.data(), mag.data() + static_cast<size_t>(j0) * out_stride, w.rows, w.cols, m,
                     out_stride);
    }
}

void oracle_gemm_d4(const HostWeight &w, const float *x, uint32_t batch, std::vector<float> &ref, uint32_t in_stride = 0,
                    uint32_t out_stride = 0) {
    in_stride = in_stride ? in_stride : w.cols;
    out_stride = out_stride ? out_stride : w.rows;
    std::vector<uint8_t> y(static_cast<size_t>(w.cols / 128) * batch * 144);
    q8o_quantize_q8_1_d4(x, batch, w.cols, in_stride, y.data());
    ref.assign(static_cast<size_t>(batch) * out_stride, 0.0f);
    q8o_gemm_d4(w.split.data(), y.data(), ref.data(), w.rows, w.cols, batch, out_stride, 8);
}

// |got - ref| <= 1e-5 |ref| + 1e-6 * sum|terms|: the allowance for a different
// fp32 summation order over the same exact per-block products
bool close_fp32(const std::vector<float> &got, const std::vector<float> &ref, const std::vector<float> &mag,
                uint32_t batch, uint32_t rows, uint32_t stride, std::string &detail) {
    for (uint32_t j = 0; j < batch; ++j)
        for (uint32_t r = 0; r < rows; ++r) {
            const size_t i = static_cast<size_t>(j) * stride + r;
            const float tol = 1e-5f * std::fabs(ref[i]) + 1e-6f * mag[i] + 1e-30f;
            if (!(std::fabs(got[i] - ref[i]) <= tol)) {
                char buf[160];
                std::snprintf(buf, sizeof(buf), "[%u,%u] got %.9g want %.9g tol %.3g", j, r, got[i], ref[i], tol);
                detail = buf;
                return false;
            }
        }
    return true;
}

bool close_abs_rel(const std::vector<float> &got, const std::vector<float> &want, float atol, float rtol,
                   std::string &detail) {
    if (got.size() != want.size()) { detail = "size mismatch"; return false; }
    for (size_t i = 0; i < got.size(); ++i) {
        if (!(std::fabs(got[i] - want[i]) <= atol + rtol * std::fabs(want[i]))) {
            char buf[128];
            std::snprintf(buf, sizeof(buf), "[%zu] got %.6g want %.6g", i, got[i], want[i]);
            detail = buf;
            return false;
        }
    }
    return true;
}

std::unique_ptr<qw3::DeviceTensor> upload_f32(qw3::HipQ8Backend &b, const std::vector<float> &v) {
    auto t = b.tensor_f32(v.size(), "t");
    if (t) require(b.copy_bytes_from_host(*t, 0, v.data(), v.size() * 4), "upload");
    return t;
}

std::vector<float> download_f32(qw3::HipQ8Backend &b, const qw3::DeviceTensor &t) {
    std::vector<float> v(t.count);
    require(b.copy_to_host(t, v.data(), 0, t.count), "download");
    return v;
}

std::vector<float> download_bf16(qw3::HipQ8Backend &b, const qw3::DeviceTensor &t) {
    std::vector<uint16_t> raw(t.count);
    require(b.copy_bytes_to_host(t, raw.data(), 0, t.count * 2), "download bf16");
    std::vector<float> v(t.count);
    for (size_t i = 0; i < v.size(); ++i) v[i] = q8o_bf16_to_f32(raw[i]);
    return v;
}

// ---- cases ----------------------------------------------------------------------------------------

// Same data and tolerances as the reference's closed-form backend test: every
// weight block is d = 0.5, q = 1; activations are constant per row.
void case_closed_form(qw3::HipQ8Backend &b) {
    constexpr uint32_t rows = 128, cols = 512, batch = 1024;
    std::vector<uint8_t> packed(static_cast<size_t>(rows) * (cols / 32) * 34);
    const uint16_t half = q8o_f32_to_f16(0.5f);
    for (size_t blk = 0; blk < packed.size() / 34; ++blk) {
        std::memcpy(&packed[blk * 34], &half, 2);
        std::memset(&packed[blk * 34 + 2], 1, 32);
    }
    auto weight = b.weight_q8_0(packed.data(), rows, cols, "w");
    std::string d;
    bool ok = weight != nullptr;

    const std::vector<float> single(cols, 0.25f);
    auto x1 = upload_f32(b, single);
    const float want1 = cols * 0.5f * 0.25f;
    auto out1 = b.tensor_bf16(rows, "o");
    ok = ok && require(b.q8_0_matvec(*out1, *weight, *x1), "matvec bf16");
    ok = ok && close_abs_rel(download_bf16(b, *out1), std::vector<float>(rows, want1), 0.1f, 0.005f, d);
    report("closed_form/matvec_bf16", ok, d);

    auto res = b.tensor_bf16(rows, "r");
    const std::vector<uint16_t> two(rows, q8o_f32_to_bf16(2.0f));
    ok = require(b.copy_bytes_from_host(*res, 0, two.data(), two.size() * 2), "copy residual");
    ok = ok && require(b.q8_0_matvec_add(*res, *weight, *x1), "matvec_add bf16");
    ok = ok && close_abs_rel(download_bf16(b, *res), std::vector<float>(rows, 2.0f + want1), 0.1f, 0.005f, d);
    report("closed_form/matvec_add_bf16", ok, d);

    std::vector<float> xin(static_cast<size_t>(batch) * cols), want(static_cast<size_t>(batch) * rows);
    for (uint32_t j = 0; j < batch; ++j) {
        const float v = static_cast<float>(j + 1) / 64.0f;
        std::fill(xin.begin() + static_cast<size_t>(j) * cols, xin.begin() + static_cast<size_t>(j + 1) * cols, v);
        std::fill(want.begin() + static_cast<size_t>(j) * rows, want.begin() + static_cast<size_t>(j + 1) * rows,
                  cols * 0.5f * v);
    }
    auto xb = upload_f32(b, xin);
    auto ob = b.tensor_bf16(want.size(), "ob");
    ok = require(b.q8_0_matmul(*ob, *weight, *xb, batch, cols, rows), "matmul bf16");
    ok = ok && close_abs_rel(download_bf16(b, *ob), want, 0.25f, 0.01f, d);
    report("closed_form/matmul_bf16_batch1024", ok, d);

    // the same in fp32: amax/127 scales make x/d exactly 127, so the result is exact
    auto of = b.tensor_f32(want.size(), "of");
    ok = require(b.q8_0_matmul(*of, *weight, *xb, batch, cols, rows), "matmul f32");
    ok = ok && close_abs_rel(download_f32(b, *of), want, 0.0f, 2e-6f, d);
    report("closed_form/matmul_f32_batch1024", ok, d);
}

void case_matvec_family(qw3::HipQ8Backend &b) {
    const uint32_t rows = 1000, cols = 2048;
    const HostWeight w = make_weight(rows, cols, 11), w2 = make_weight(rows, cols, 12);
    auto dw = b.weight_q8_0(w.gguf.data(), rows, cols, "w");
    auto dw2 = b.weight_q8_0(w2.gguf.data(), rows, cols, "w2");
    const auto x = normal_vec(cols, 13);
    auto dx = upload_f32(b, x);
    std::vector<float> ref, mag, ref2, mag2;
    oracle_linear(w, x.data(), 1, cols, rows, ref, mag);
    oracle_linear(w2, x.data(), 1, cols, rows, ref2, mag2);
    std::string d;

    auto out = b.tensor_f32(rows, "o");
    bool ok = require(b.q8_0_matvec(*out, *dw, *dx), "matvec");
    ok = ok && close_fp32(download_f32(b, *out), ref, mag, 1, rows, rows, d);
    report("matvec_f32", ok, d);

    const auto base = normal_vec(rows, 14);
    auto acc = upload_f32(b, base);
    ok = require(b.q8_0_matvec_add(*acc, *dw, *dx), "matvec_add");
    std::vector<float> want(rows), magadd(rows);
    for (uint32_t r = 0; r < rows; ++r) { want[r] = base[r] + ref[r]; magadd[r] = mag[r] + std::fabs(base[r]); }
    ok = ok && close_fp32(download_f32(b, *acc), want, magadd, 1, rows, rows, d);
    report("matvec_add_f32", ok, d);

    // silu(g) * u: compared against the oracle's own fused form; tolerance widened
    // by the derivative bound |silu'| <= 1.1 and one ulp of expf
    std::vector<uint8_t> y(static_cast<size_t>(cols / 32) * 36);
    q8o_quantize_q8_1(x.data(), 1, cols, cols, y.data());
    std::vector<float> silu(rows);
    q8o_gemv_silu_mul(w.split.data(), w2.split.data(), y.data(), silu.data(), rows, cols, 1, rows);
    ok = require(b.q8_0_matvec_silu_mul(*out, *dw, *dw2, *dx), "silu_mul");
    {
        const auto got = download_f32(b, *out);
        for (uint32_t r = 0; r < rows && ok; ++r) {
            const float tg = 1e-5f * std::fabs(ref[r]) + 1e-6f * mag[r];
            const float tu = 1e-5f * std::fabs(ref2[r]) + 1e-6f * mag2[r];
            const float tol = 1.1f * tg * std::fabs(ref2[r]) + tu * std::fabs(ref[r]) + 4e-7f * std::fabs(silu[r]) +
                              1e-30f;
            if (!(std::fabs(got[r] - silu[r]) <= tol)) {
                char buf[128];
                std::snprintf(buf, sizeof(buf), "[%u] got %.9g want %.9g tol %.3g", r, got[r], silu[r], tol);
                d = buf;
                ok = false;
            }
        }
    }
    report("matvec_silu_mul", ok, d);

    // fan-out: three weights of different heights sharing one activation
    const HostWeight wa = make_weight(768, cols, 21), wb = make_weight(130, cols, 22), wc = make_weight(31, cols, 23);
    auto da = b.weight_q8_0(wa.gguf.data(), wa.rows, cols, "a");
    auto db = b.weight_q8_0(wb.gguf.data(), wb.rows, cols, "b");
    auto dc = b.weight_q8_0(wc.gguf.data(), wc.rows, cols, "c");
    auto oa = b.tensor_f32(wa.rows, "oa"), ob = b.tensor_f32(wb.rows, "ob"), oc = b.tensor_f32(wc.rows, "oc");
    qw3::DeviceTensor *outs[3] = {oa.get(), ob.get(), oc.get()};
    const qw3::DeviceWeight *ws[3] = {da.get(), db.get(), dc.get()};
    ok = require(b.q8_0_matvec_fanout(outs, ws, 3, *dx), "fanout");
    const HostWeight *hw[3] = {&wa, &wb, &wc};
    for (int i = 0; i < 3 && ok; ++i) {
        oracle_linear(*hw[i], x.data(), 1, cols, hw[i]->rows, ref, mag);
        ok = close_fp32(download_f32(b, *outs[i]), ref, mag, 1, hw[i]->rows, hw[i]->rows, d);
    }
    report("matvec_fanout3", ok, d);

    // format-neutral forwards: the same operators under the names the executor calls
    auto la = b.tensor_f32(wa.rows, "la"), lb = b.tensor_f32(wb.rows, "lb"), lc = b.tensor_f32(wc.rows, "lc");
    qw3::DeviceTensor *louts[3] = {la.get(), lb.get(), lc.get()};
    ok = require(b.linear_matvec_fanout(louts, ws, 3, *dx), "linear_matvec_fanout");
    for (int i = 0; i < 3 && ok; ++i) {
        oracle_linear(*hw[i], x.data(), 1, cols, hw[i]->rows, ref, mag);
        ok = close_fp32(download_f32(b, *louts[i]), ref, mag, 1, hw[i]->rows, hw[i]->rows, d);
    }
    auto lo = b.tensor_f32(rows, "lo");
    ok = ok && require(b.linear_matvec(*lo, *dw, *dx), "linear_matvec") && require(b.q8_0_matvec(*out, *dw, *dx), "matvec");
    ok = ok && download_f32(b, *lo) == download_f32(b, *out);
    ok = ok && require(b.linear_matmul(*lo, *dw, *dx, 1, cols, rows), "linear_matmul");
    oracle_linear(w, x.data(), 1, cols, rows, ref, mag);
    ok = ok && close_fp32(download_f32(b, *lo), ref, mag, 1, rows, rows, d);
    report("linear_forwards", ok, d);
}

void case_matmul(qw3::HipQ8Backend &b) {
    std::string d;
    // batch <= 8 and strided batches: GEMV route, bit-for-bit the Q8_1 quantizer
    {
        const uint32_t rows = 515, cols = 1024;
        const HostWeight w = make_weight(rows, cols, 31);
        auto dw = b.weight_q8_0(w.gguf.data(), rows, cols, "w");
        for (uint32_t batch : {2u, 5u, 8u, 19u}) {
            const uint32_t in_stride = cols + 64, out_stride = rows + 9;
            const auto x = normal_vec(static_cast<size_t>(batch) * in_stride, 32 + batch);
            auto dx = upload_f32(b, x);
            auto out = b.tensor_f32(static_cast<size_t>(batch) * out_stride, "o");
            require(b.zero_tensor(*out), "zero");
            bool ok = require(b.q8_0_matmul(*out, *dw, *dx, batch, in_stride, out_stride), "matmul strided");
            std::vector<float> ref, mag;
            oracle_linear(w, x.data(), batch, in_stride, out_stride, ref, mag);
            const auto got = download_f32(b, *out);
            ok = ok && close_fp32(got, ref, mag, batch, rows, out_stride, d);
            for (uint32_t j = 0; j < batch && ok; ++j)     // the gap between rows stays untouched
                for (uint32_t r = rows; r < out_stride; ++r)
                    if (got[static_cast<size_t>(j) * out_stride + r] != 0.0f) { ok = false; d = "wrote into the stride gap"; }
            report(("matmul_strided_batch" + std::to_string(batch)).c_str(), ok, d);
        }
    }
    // contiguous batch > 8, D4 layout: MFMA tile (and its medium-batch variant)
    {
        const uint32_t rows = 384, cols = 1024;
        const HostWeight w = make_weight(rows, cols, 41);
        auto dw = b.weight_q8_0(w.gguf.data(), rows, cols, "w");
        for (uint32_t batch : {9u, 16u, 64u, 65u, 300u}) {
            const auto x = normal_vec(static_cast<size_t>(batch) * cols, 42 + batch);
            auto dx = upload_f32(b, x);
            auto out = b.tensor_f32(static_cast<size_t>(batch) * rows, "o");
            bool ok = require(b.q8_0_matmul(*out, *dw, *dx, batch, cols, rows), "matmul d4");
            std::vector<float> ref, lin, mag;
            oracle_gemm_d4(w, x.data(), batch, ref);
            oracle_linear(w, x.data(), batch, cols, rows, lin, mag);   // magnitudes only
            ok = ok && close_fp32(download_f32(b, *out), ref, mag, batch, rows, rows, d);
            report(("matmul_d4_batch" + std::to_string(batch)).c_str(), ok, d);
        }
    }
    // contiguous batch > 8 where the layout rule keeps Q8_1 (rows < 128, cols % 128 != 0)
    {
        const uint32_t rows = 100, cols = 480, batch = 40;
        const HostWeight w = make_weight(rows, cols, 51);
        auto dw = b.weight_q8_0(w.gguf.data(), rows, cols, "w");
        const auto x = normal_vec(static_cast<size_t>(batch) * cols, 52);
        auto dx = upload_f32(b, x);
        auto out = b.tensor_f32(static_cast<size_t>(batch) * rows, "o");
        bool ok = require(b.q8_0_matmul(*out, *dw, *dx, batch, cols, rows), "matmul q8_1 layout");
        std::vector<float> ref, mag;
        oracle_linear(w, x.data(), batch, cols, rows, ref, mag);
        ok = ok && close_fp32(download_f32(b, *out), ref, mag, batch, rows, rows, d);
        report("matmul_q8_1_layout_batch40", ok, d);
    }
    // fan-out at batch 4 and in-place residual add at batch 3
    {
        const uint32_t cols = 768, batch = 4;
        const HostWeight wa = make_weight(256, cols, 61), wb = make_weight(64, cols, 62);
        auto da = b.weight_q8_0(wa.gguf.data(), wa.rows, cols, "a");
        auto db = b.weight_q8_0(wb.gguf.data(), wb.rows, cols, "b");
        const auto x = normal_vec(static_cast<size_t>(batch) * cols, 63);
        auto dx = upload_f32(b, x);
        const uint32_t strides[2] = {300, 64};
        auto oa = b.tensor_f32(batch * strides[0], "oa"), ob = b.tensor_f32(batch * strides[1], "ob");
        qw3::DeviceTensor *outs[2] = {oa.get(), ob.get()};
        const qw3::DeviceWeight *ws[2] = {da.get(), db.get()};
        bool ok = require(b.q8_0_matmul_fanout(outs, ws, strides, 2, *dx, batch, cols), "matmul_fanout");
        std::vector<float> ref, mag;
        oracle_linear(wa, x.data(), batch, cols, strides[0], ref, mag);
        ok = ok && close_fp32(download_f32(b, *oa), ref, mag, batch, wa.rows, strides[0], d);
        oracle_linear(wb, x.data(), batch, cols, strides[1], ref, mag);
        ok = ok && close_fp32(download_f32(b, *ob), ref, mag, batch, wb.rows, strides[1], d);
        report("matmul_fanout_batch4", ok, d);

        const uint32_t nb = 3;
        const auto base = normal_vec(static_cast<size_t>(nb) * wa.rows, 64);
        auto acc = upload_f32(b, base);
        auto tmp = b.tensor_f32(1, "tmp");
        ok = require(b.q8_0_matmul_add(*acc, *acc, *tmp, *da, *dx, nb, cols, wa.rows), "matmul_add");
        oracle_linear(wa, x.data(), nb, cols, wa.rows, ref, mag);
        for (size_t i = 0; i < ref.size(); ++i) { ref[i] += base[i]; mag[i] += std::fabs(base[i]); }
        ok = ok && close_fp32(download_f32(b, *acc), ref, mag, nb, wa.rows, wa.rows, d);
        report("matmul_add_inplace_batch3", ok, d);

        // out of place at batch 3 (no fused form): matmul into the temporary, then out = residual + tmp
        {
            auto other = b.tensor_f32(static_cast<size_t>(nb) * wa.rows, "other");
            auto tmp3 = b.tensor_f32(static_cast<size_t>(nb) * wa.rows, "tmp3");
            auto res = upload_f32(b, base);
            ok = require(b.q8_0_matmul_add(*other, *res, *tmp3, *da, *dx, nb, cols, wa.rows), "matmul_add out of place");
            oracle_linear(wa, x.data(), nb, cols, wa.rows, ref, mag);
            for (size_t i = 0; i < ref.size(); ++i) { ref[i] = base[i] + ref[i]; mag[i] += std::fabs(base[i]); }
            ok = ok && close_fp32(download_f32(b, *other), ref, mag, nb, wa.rows, wa.rows, d);
            ok = ok && download_f32(b, *res) == base;    // the residual is left alone
            report("matmul_add_out_of_place_batch3", ok, d);
        }
        // forms the backend declines, as the reference does
        auto other = b.tensor_f32(static_cast<size_t>(nb) * wa.rows, "other");
        ok = !b.q8_0_matmul_silu_mul(*other, *da, *db, *dx, nb, cols, wa.rows).ok;   // gate / up heights differ
        ok = ok && !b.q8_0_matmul_silu_mul(*other, *da, *da, *dx, nb, cols - 1, wa.rows).ok;   // stride shorter than a row
        ok = ok && b.weight_q8_0(wa.gguf.data(), 4, 40, "bad") == nullptr;
        ok = ok && !b.add_n(*other, *other, *other, other->count + 1).ok;
        ok = ok && !b.silu_mul_n(*other, *other, *other, other->count + 1).ok;
        report("declined_forms", ok);
    }
}

// Batched q8_0_matmul_add beyond the fused in-place form (src/kernels_cuda.cu:11919-11957 falls back to
// include/qw3/device_backend.hpp:529-540: q8_0_matmul into matmul_tmp, then add): batch 9, 64 and 2048,
// in place (out == residual) and out of place, fp32; and bf16 tensors at batch 64.
void case_matmul_add_batched(qw3::HipQ8Backend &b) {
    std::string d;
    const uint32_t rows = 384, cols = 1024;
    const HostWeight w = make_weight(rows, cols, 141);
    auto dw = b.weight_q8_0(w.gguf.data(), rows, cols, "w");
    for (uint32_t batch : {9u, 64u, 2048u}) {
        const auto x = normal_vec(static_cast<size_t>(batch) * cols, 142 + batch);
        const auto base = normal_vec(static_cast<size_t>(batch) * rows, 143 + batch);
        auto dx = upload_f32(b, x);
        std::vector<float> prod, lin, mag;
        oracle_gemm_d4(w, x.data(), batch, prod);                  // what q8_0_matmul leaves in the temporary
        oracle_linear(w, x.data(), batch, cols, rows, lin, mag);   // magnitudes only
        std::vector<float> want(prod.size());
        for (size_t i = 0; i < prod.size(); ++i) { want[i] = base[i] + prod[i]; mag[i] += std::fabs(base[i]); }
        for (int in_place = 0; in_place < 2; ++in_place) {
            auto res = upload_f32(b, base);
            auto tmp = b.tensor_f32(static_cast<size_t>(batch) * rows, "tmp");
            auto other = b.tensor_f32(static_cast<size_t>(batch) * rows, "out");
            qw3::DeviceTensor &out = in_place ? *res : *other;
            bool ok = require(b.q8_0_matmul_add(out, *res, *tmp, *dw, *dx, batch, cols, rows), "matmul_add batched");
            ok = ok && close_fp32(download_f32(b, out), want, mag, batch, rows, rows, d);
            if (!in_place) ok = ok && download_f32(b, *res) == base;
            report(("matmul_add_batch" + std::to_string(batch) + (in_place ? "_in_place" : "_out_of_place")).c_str(), ok, d);
        }
    }
    // bf16 tensors: the temporary is the product rounded to bf16, the sum is rounded again
    {
        const uint32_t batch = 64;
        const auto x = normal_vec(static_cast<size_t>(batch) * cols, 151);
        auto dx = upload_f32(b, x);
        std::vector<float> prod;
        oracle_gemm_d4(w, x.data(), batch, prod);
        const auto basef = normal_vec(static_cast<size_t>(batch) * rows, 152);
        std::vector<uint16_t> base(basef.size());
        for (size_t i = 0; i < base.size(); ++i) base[i] = q8o_f32_to_bf16(basef[i]);
        auto res = b.tensor_bf16(base.size(), "res"), tmp = b.tensor_bf16(base.size(), "tmp"), out = b.tensor_bf16(base.size(), "out");
        bool ok = res && tmp && out && require(b.copy_bytes_from_host(*res, 0, base.data(), base.size() * 2), "upload bf16");
        ok = ok && require(b.q8_0_matmul_add(*out, *res, *tmp, *dw, *dx, batch, cols, rows), "matmul_add bf16");
        std::vector<uint16_t> got(base.size()), mid(base.size());
        ok = ok && require(b.copy_bytes_to_host(*out, got.data(), 0, got.size() * 2), "download bf16");
        ok = ok && require(b.copy_bytes_to_host(*tmp, mid.data(), 0, mid.size() * 2), "download bf16 tmp");
        // the temporary: the oracle's product rounded to bf16, or its neighbour where the GPU's fp32 sum
        // (same terms, another order) lies across a rounding boundary; the output: exactly the rounded
        // sum of the residual and that temporary
        size_t off = 0, far = 0;
        for (size_t i = 0; i < got.size(); ++i) {
            const int diff = std::abs(static_cast<int>(mid[i]) - static_cast<int>(q8o_f32_to_bf16(prod[i])));
            off += diff != 0;
            far += diff > 1;
            if (got[i] != q8o_f32_to_bf16(q8o_bf16_to_f32(base[i]) + q8o_bf16_to_f32(mid[i]))) ++far;
        }
        ok = ok && far == 0 && off * 100 < got.size();
        report("matmul_add_bf16_batch64", ok, "differing " + std::to_string(off) + ", beyond one step " + std::to_string(far));
    }
}

// silu(g) * u for sums g, u that are each within the GEMV / GEMM tolerance (tg, tu) of their
// references: the derivative bound |silu'| <= 1.1 and a few ulp of the fast exponential.
bool close_swiglu(const std::vector<float> &got, const std::vector<float> &gref, const std::vector<float> &gmag,
                  const std::vector<float> &uref, const std::vector<float> &umag, uint32_t batch, uint32_t rows,
                  uint32_t stride, std::string &detail) {
    for (uint32_t j = 0; j < batch; ++j)
        for (uint32_t r = 0; r < rows; ++r) {
            const size_t i = static_cast<size_t>(j) * stride + r;
            const double g = gref[i], u = uref[i];
            const double want = g / (1.0 + std::exp(-g)) * u;
            const double tg = 1e-5 * std::fabs(g) + 1e-6 * gmag[i], tu = 1e-5 * std::fabs(u) + 1e-6 * umag[i];
            const double tol = 1.1 * tg * std::fabs(u) + tu * std::fabs(g) + 1e-6 * std::fabs(want) + 1e-30;
            if (!(std::fabs(got[i] - want) <= tol)) {
                char buf[160];
                std::snprintf(buf, sizeof(buf), "[%u,%u] got %.9g want %.9g tol %.3g", j, r, got[i], want, tol);
                detail = buf;
                return false;
            }
        }
    return true;
}

// q8_0_matmul_silu_mul (include/qw3/device_backend.hpp:330-336) for Q8_0 at every batch regime: GEMV
// (2, 8, strided), matrix-core GEMV on D4 records (9, 16), ring tiles (20, 40, 64, 300) and main tiles
// (512 x 3328 rows, and ragged 500 x 3300), against the oracle's two products (Q8_1 rows up to eight,
// D4 records above: the quantizer each route uses) combined in double; and silu_mul / silu_mul_n.
void case_silu_mul(qw3::HipQ8Backend &b) {
    std::string d;
    auto run = [&](uint32_t rows, uint32_t cols, uint32_t batch, uint32_t in_stride, uint32_t out_stride, uint64_t seed) {
        d.clear();
        const HostWeight wg = make_weight(rows, cols, seed), wu = make_weight(rows, cols, seed + 1);
        auto dg = b.weight_q8_0(wg.gguf.data(), rows, cols, "g");
        auto du = b.weight_q8_0(wu.gguf.data(), rows, cols, "u");
        const auto x = normal_vec(static_cast<size_t>(batch) * in_stride, seed + 2);
        auto dx = upload_f32(b, x);
        auto out = b.tensor_f32(static_cast<size_t>(batch) * out_stride, "o");
        bool ok = dg && du && require(b.zero_tensor(*out), "zero");
        ok = ok && require(b.q8_0_matmul_silu_mul(*out, *dg, *du, *dx, batch, in_stride, out_stride), "matmul_silu_mul");
        std::vector<float> gref, gmag, uref, umag;
        oracle_linear(wg, x.data(), batch, in_stride, out_stride, gref, gmag);
        oracle_linear(wu, x.data(), batch, in_stride, out_stride, uref, umag);
        if (batch > 8 && rows >= 128 && cols % 256 == 0) {   // D4 records
            oracle_gemm_d4(wg, x.data(), batch, gref, in_stride, out_stride);
            oracle_gemm_d4(wu, x.data(), batch, uref, in_stride, out_stride);
        }
        const auto got = download_f32(b, *out);
        ok = ok && close_swiglu(got, gref, gmag, uref, umag, batch, rows, out_stride, d);
        for (uint32_t j = 0; j < batch && ok; ++j)     // the gap between rows stays untouched
            for (uint32_t r = rows; r < out_stride; ++r)
                if (got[static_cast<size_t>(j) * out_stride + r] != 0.0f) { ok = false; d = "wrote into the stride gap"; }
        char name[96];
        std::snprintf(name, sizeof(name), "matmul_silu_mul_%ux%u_batch%u%s", rows, cols, batch,
                      (in_stride != cols || out_stride != rows) ? "_strided" : "");
        report(name, ok, d);
    };
    for (uint32_t batch : {1u, 2u, 8u, 9u, 16u, 20u, 40u, 64u, 300u}) run(384, 1024, batch, 1024, 384, 500 + batch);
    run(384, 1024, 5, 1024 + 32, 384 + 8, 520);       // strided GEMV route
    run(384, 1024, 19, 1024 + 32, 384 + 8, 521);      // strided above eight rows: the tiles take strides
    run(200, 480, 12, 480, 200, 522);                 // cols % 128 != 0: GEMV slices
    run(3328, 512, 512, 512, 3328, 523);              // 64 + 64-row main tiles
    run(3300, 512, 500, 512, 3300, 524);              // the same with ragged edges

    // elementwise silu_mul / silu_mul_n on a length that is not a multiple of four
    {
        const size_t n = 4099, part = 1030;
        const auto g = normal_vec(n, 530, 3.0f), u = normal_vec(n, 531);
        auto dg = upload_f32(b, g), du = upload_f32(b, u);
        auto out = b.tensor_f32(n, "o");
        bool ok = require(b.zero_tensor(*out), "zero") && require(b.silu_mul_n(*out, *dg, *du, part), "silu_mul_n");
        auto got = download_f32(b, *out);
        auto check = [&](size_t upto) {
            for (size_t i = 0; i < n && ok; ++i) {
                const double want = i < upto ? static_cast<double>(g[i]) / (1.0 + std::exp(-static_cast<double>(g[i]))) * u[i] : 0.0;
                if (!(std::fabs(got[i] - want) <= 1e-6 * std::fabs(want))) { ok = false; d = "element " + std::to_string(i); }
            }
        };
        check(part);
        ok = ok && require(b.silu_mul(*out, *dg, *du), "silu_mul");
        got = download_f32(b, *out);
        check(n);
        report("silu_mul_n", ok, d);
    }
}

// A norm and the projection that reads its output share a launch (one row) or the quantized rows
// (up to eight); whatever a caller does in between, the results are the bits of the separate steps.
void case_norm_reuse(qw3::HipQ8Backend &b) {
    std::string d;
    const uint32_t cols = 2048, rows = 640;
    const float eps = 1e-6f;
    const HostWeight w = make_weight(rows, cols, 601), w2 = make_weight(rows, cols, 602), wd = make_weight(cols, rows, 603);
    auto dw = b.weight_q8_0(w.gguf.data(), rows, cols, "w");
    auto dw2 = b.weight_q8_0(w2.gguf.data(), rows, cols, "w2");
    auto nwv = normal_vec(cols, 604, 0.4f);
    for (auto &f : nwv) f += 1.0f;
    auto nw = b.weight_f32(nwv.data(), cols, "norm.weight");
    auto bits_equal = [](const std::vector<float> &a, const std::vector<float> &c) {
        return a.size() == c.size() && std::memcmp(a.data(), c.data(), a.size() * 4) == 0;
    };
    for (uint32_t batch : {1u, 3u}) {
        const auto x = normal_vec(static_cast<size_t>(batch) * cols, 610 + batch, 2.0f);
        auto dx = upload_f32(b, x);
        std::vector<float> nref(x.size());
        q8o_rms_norm(x.data(), nwv.data(), nref.data(), batch, cols, cols, cols, eps);
        auto norm_a = b.tensor_f32(x.size(), "na"), norm_b = b.tensor_f32(x.size(), "nb");
        auto oa = b.tensor_f32(static_cast<size_t>(batch) * rows, "oa"), ob = b.tensor_f32(static_cast<size_t>(batch) * rows, "ob");
        auto sa = b.tensor_f32(static_cast<size_t>(batch) * rows, "sa"), sb = b.tensor_f32(static_cast<size_t>(batch) * rows, "sb");
        // back to back: the projection may take the norm into its launch / read the norm's blocks
        bool ok = require(b.rms_norm_batch(*norm_a, *dx, *nw, batch, cols, eps), "norm") &&
                  require(b.q8_0_matmul(*oa, *dw, *norm_a, batch, cols, rows), "matmul after norm") &&
                  require(b.rms_norm_batch(*norm_a, *dx, *nw, batch, cols, eps), "norm") &&
                  require(b.q8_0_matmul_silu_mul(*sa, *dw, *dw2, *norm_a, batch, cols, rows), "silu after norm");
        // with a synchronisation in between: separate launches
        ok = ok && require(b.rms_norm_batch(*norm_b, *dx, *nw, batch, cols, eps), "norm") && require(b.synchronize(), "sync") &&
             require(b.zero_tensor(*ob), "zero") &&
             require(b.q8_0_matmul(*ob, *dw, *norm_b, batch, cols, rows), "matmul") &&
             require(b.zero_tensor(*sb), "zero") &&
             require(b.q8_0_matmul_silu_mul(*sb, *dw, *dw2, *norm_b, batch, cols, rows), "silu");
        ok = ok && bits_equal(download_f32(b, *norm_a), nref) && bits_equal(download_f32(b, *norm_b), nref);
        ok = ok && bits_equal(download_f32(b, *oa), download_f32(b, *ob)) && bits_equal(download_f32(b, *sa), download_f32(b, *sb));
        std::vector<float> ref, mag;
        oracle_linear(w, nref.data(), batch, cols, rows, ref, mag);
        ok = ok && close_fp32(download_f32(b, *oa), ref, mag, batch, rows, rows, d);
        report(("norm_then_projection_batch" + std::to_string(batch)).c_str(), ok, d);

        // the normalised rows change between two projections: the second must see the new rows
        std::vector<float> other = normal_vec(x.size(), 620 + batch);
        ok = require(b.rms_norm_batch(*norm_a, *dx, *nw, batch, cols, eps), "norm") &&
             require(b.q8_0_matmul(*oa, *dw, *norm_a, batch, cols, rows), "matmul") &&
             require(b.copy_bytes_from_host(*norm_a, 0, other.data(), other.size() * 4), "overwrite") &&
             require(b.q8_0_matmul(*oa, *dw, *norm_a, batch, cols, rows), "matmul again");
        oracle_linear(w, other.data(), batch, cols, rows, ref, mag);
        ok = ok && close_fp32(download_f32(b, *oa), ref, mag, batch, rows, rows, d);
        // ... also when a projection itself overwrites them (its output is the norm's output tensor)
        auto sq = b.tensor_f32(static_cast<size_t>(batch) * cols, "sq");
        auto dwd = b.weight_q8_0(wd.gguf.data(), cols, rows, "wd");
        ok = ok && require(b.rms_norm_batch(*norm_a, *dx, *nw, batch, cols, eps), "norm") &&
             require(b.q8_0_matmul(*oa, *dw, *norm_a, batch, cols, rows), "matmul") &&
             require(b.q8_0_matmul(*norm_a, *dwd, *oa, batch, rows, cols), "matmul into the norm's tensor") &&
             require(b.q8_0_matmul(*ob, *dw, *norm_a, batch, cols, rows), "matmul of the new rows");
        const auto mid = download_f32(b, *norm_a);
        oracle_linear(w, mid.data(), batch, cols, rows, ref, mag);
        ok = ok && close_fp32(download_f32(b, *ob), ref, mag, batch, rows, rows, d);
        report(("norm_rows_overwritten_batch" + std::to_string(batch)).c_str(), ok, d);
    }
    // one row, a projection that writes the norm's input: the norm must run first
    {
        const auto x = normal_vec(cols, 630, 2.0f);
        auto h = upload_f32(b, x);
        std::vector<float> nref(cols);
        q8o_rms_norm(x.data(), nwv.data(), nref.data(), 1, cols, cols, cols, eps);
        auto norm = b.tensor_f32(cols, "n");
        const HostWeight wsq = make_weight(cols, cols, 631);
        auto dsq = b.weight_q8_0(wsq.gguf.data(), cols, cols, "sq");
        bool ok = require(b.rms_norm(*norm, *h, *nw, eps), "norm") && require(b.q8_0_matvec(*h, *dsq, *norm), "matvec into the norm's input");
        std::vector<float> ref, mag;
        oracle_linear(wsq, nref.data(), 1, cols, cols, ref, mag);
        ok = ok && close_fp32(download_f32(b, *h), ref, mag, 1, cols, cols, d) && bits_equal(download_f32(b, *norm), nref);
        report("norm_input_overwritten_by_projection", ok, d);
    }
    // a held-back norm inside a captured graph: replays equal the eager run
    {
        const auto x = normal_vec(cols, 640, 2.0f);
        auto h = upload_f32(b, x);
        auto norm = b.tensor_f32(cols, "n");
        auto out = b.tensor_f32(rows, "o");
        auto step = [&]() { return b.rms_norm(*norm, *h, *nw, eps).ok && b.q8_0_matvec_silu_mul(*out, *dw, *dw2, *norm).ok; };
        bool ok = step() && require(b.synchronize(), "sync");
        const auto eager = download_f32(b, *out);
        ok = ok && b.begin_capture() && step();
        ok = require(b.end_capture(), "end_capture") && ok;
        for (int rep = 0; rep < 3 && ok; ++rep) {
            ok = require(b.zero_tensor(*out), "zero") && require(b.zero_tensor(*norm), "zero") && require(b.replay_graph(), "replay") &&
                 require(b.synchronize(), "sync");
            ok = ok && bits_equal(download_f32(b, *out), eager);
        }
        // ... and a norm left pending when the capture ends is part of the graph
        ok = ok && b.begin_capture() && b.rms_norm(*norm, *h, *nw, eps).ok;
        ok = require(b.end_capture(), "end_capture") && ok;
        std::vector<float> nref(cols);
        q8o_rms_norm(x.data(), nwv.data(), nref.data(), 1, cols, cols, cols, eps);
        ok = ok && require(b.zero_tensor(*norm), "zero") && require(b.replay_graph(), "replay") && bits_equal(download_f32(b, *norm), nref);
        report("norm_held_back_under_capture", ok);
    }
    // tensors destroyed while a norm is held back: an output nobody can read is dropped, an input
    // is read before it is freed
    {
        const auto x = normal_vec(cols, 645, 2.0f);
        std::vector<float> nref(cols);
        q8o_rms_norm(x.data(), nwv.data(), nref.data(), 1, cols, cols, cols, eps);
        auto h = upload_f32(b, x);
        auto gone = b.tensor_f32(cols, "gone");
        bool ok = require(b.rms_norm(*gone, *h, *nw, eps), "norm into a tensor about to go");
        gone.reset();
        auto norm = b.tensor_f32(cols, "n");
        ok = ok && require(b.rms_norm(*norm, *h, *nw, eps), "norm");
        h.reset();                                  // the norm's input goes: the norm runs first
        ok = ok && bits_equal(download_f32(b, *norm), nref);
        auto out = b.tensor_f32(rows, "o");
        ok = ok && require(b.q8_0_matvec(*out, *dw, *norm), "matvec after the tensors went");
        std::vector<float> ref, mag;
        oracle_linear(w, nref.data(), 1, cols, rows, ref, mag);
        ok = ok && close_fp32(download_f32(b, *out), ref, mag, 1, rows, rows, d);
        report("norm_held_back_tensors_destroyed", ok, d);
    }
    // the shortcuts switched off (a host whose other kernels write these tensors): same bits
    for (uint32_t batch : {1u, 4u}) {
        const auto x = normal_vec(static_cast<size_t>(batch) * cols, 650 + batch, 2.0f);
        auto dx = upload_f32(b, x);
        auto norm = b.tensor_f32(x.size(), "n");
        auto on = b.tensor_f32(static_cast<size_t>(batch) * rows, "on"), off = b.tensor_f32(static_cast<size_t>(batch) * rows, "off");
        bool ok = require(b.rms_norm_batch(*norm, *dx, *nw, batch, cols, eps), "norm") &&
                  require(b.q8_0_matmul_silu_mul(*on, *dw, *dw2, *norm, batch, cols, rows), "silu, shortcuts on");
        b.set_norm_shortcuts(false);
        ok = ok && !b.norm_shortcuts() && require(b.rms_norm_batch(*norm, *dx, *nw, batch, cols, eps), "norm") &&
             require(b.q8_0_matmul_silu_mul(*off, *dw, *dw2, *norm, batch, cols, rows), "silu, shortcuts off");
        b.set_norm_shortcuts(true);
        ok = ok && bits_equal(download_f32(b, *on), download_f32(b, *off));
        // invalidate_norm_state() runs a held-back norm: its output is there before any projection
        std::vector<float> nref(x.size());
        q8o_rms_norm(x.data(), nwv.data(), nref.data(), batch, cols, cols, cols, eps);
        ok = ok && require(b.zero_tensor(*norm), "zero") && require(b.rms_norm_batch(*norm, *dx, *nw, batch, cols, eps), "norm") &&
             require(b.invalidate_norm_state(), "invalidate") && bits_equal(download_f32(b, *norm), nref);
        report(("norm_shortcuts_off_batch" + std::to_string(batch)).c_str(), ok);
    }
}

// add / add_n held back for the norm of its sum (the batched layer loop's add_n + rms_norm_batch):
// the sum, the normalised rows and the projection behind them are the bits of the separate
// launches, whatever call comes next.
void case_add_held_back(qw3::HipQ8Backend &b) {
    std::string d;
    const uint32_t cols = 2048, rows = 640;
    const float eps = 1e-6f;
    const HostWeight w = make_weight(rows, cols, 701);
    auto dw = b.weight_q8_0(w.gguf.data(), rows, cols, "w");
    auto nwv = normal_vec(cols, 704, 0.4f);
    for (auto &f : nwv) f += 1.0f;
    auto nw = b.weight_f32(nwv.data(), cols, "norm.weight");
    auto bits_equal = [](const std::vector<float> &a, const std::vector<float> &c) {
        return a.size() == c.size() && std::memcmp(a.data(), c.data(), a.size() * 4) == 0;
    };
    for (uint32_t batch : {1u, 2u, 8u, 9u, 40u}) {
        const size_t n = static_cast<size_t>(batch) * cols;
        const auto hv = normal_vec(n, 710 + batch, 2.0f), dv = normal_vec(n, 720 + batch, 0.7f);
        std::vector<float> sum(n), nref(n);
        for (size_t i = 0; i < n; ++i) sum[i] = hv[i] + dv[i];
        q8o_rms_norm(sum.data(), nwv.data(), nref.data(), batch, cols, cols, cols, eps);
        std::vector<float> ref, mag;
        oracle_linear(w, nref.data(), batch, cols, rows, ref, mag);
        auto delta = upload_f32(b, dv);
        auto norm = b.tensor_f32(n, "n");
        auto out = b.tensor_f32(static_cast<size_t>(batch) * rows, "o");
        std::vector<float> first_out;
        for (int shortcuts = 1; shortcuts >= 0; --shortcuts) {
            b.set_norm_shortcuts(shortcuts != 0);
            auto h = upload_f32(b, hv);
            bool ok = require(b.zero_tensor(*norm), "zero") && require(b.add_n(*h, *h, *delta, n), "add_n in place") &&
                      require(b.rms_norm_batch(*norm, *h, *nw, batch, cols, eps), "norm of the sum") &&
                      require(b.q8_0_matmul(*out, *dw, *norm, batch, cols, rows), "projection");
            ok = ok && bits_equal(download_f32(b, *h), sum) && bits_equal(download_f32(b, *norm), nref);
            const auto got = download_f32(b, *out);
            if (batch <= 8) ok = ok && close_fp32(got, ref, mag, batch, rows, rows, d);
            if (shortcuts) first_out = got;
            else ok = ok && bits_equal(got, first_out);
            report(("add_then_norm_batch" + std::to_string(batch) + (shortcuts ? "" : "_shortcuts_off")).c_str(), ok, d);
        }
        b.set_norm_shortcuts(true);
        // the same in front of the fused norm + fan-out operator (the add_n that ends a layer, then the next layer's first call)
        std::vector<float> first_fan;
        for (int shortcuts = 1; shortcuts >= 0; --shortcuts) {
            b.set_norm_shortcuts(shortcuts != 0);
            auto h = upload_f32(b, hv);
            qw3::DeviceTensor *outs[1] = {out.get()};
            const qw3::DeviceWeight *ws[1] = {dw.get()};
            const uint32_t strides[1] = {rows};
            bool ok = require(b.zero_tensor(*norm), "zero") && require(b.zero_tensor(*out), "zero") &&
                      require(b.add_n(*h, *h, *delta, n), "add_n in place") &&
                      require(b.rms_norm_q8_0_matmul_fanout(*norm, outs, ws, strides, 1, *h, *nw, batch, cols, eps), "norm + fan-out of the sum");
            ok = ok && bits_equal(download_f32(b, *h), sum) && bits_equal(download_f32(b, *norm), nref);
            const auto got = download_f32(b, *out);
            if (batch <= 8) ok = ok && close_fp32(got, ref, mag, batch, rows, rows, d);
            if (shortcuts) first_fan = got;
            else ok = ok && bits_equal(got, first_fan);
            report(("add_then_norm_fanout_batch" + std::to_string(batch) + (shortcuts ? "" : "_shortcuts_off")).c_str(), ok, d);
        }
        b.set_norm_shortcuts(true);
    }
    {
        const uint32_t batch = 4;
        const size_t n = static_cast<size_t>(batch) * cols;
        const auto hv = normal_vec(n, 731, 2.0f), dv = normal_vec(n, 732, 0.7f);
        std::vector<float> sum(n), nref(n), nplain(n);
        for (size_t i = 0; i < n; ++i) sum[i] = hv[i] + dv[i];
        q8o_rms_norm(sum.data(), nwv.data(), nref.data(), batch, cols, cols, cols, eps);
        q8o_rms_norm(hv.data(), nwv.data(), nplain.data(), batch, cols, cols, cols, eps);
        auto delta = upload_f32(b, dv);
        // out of place, and read back right away: the add runs before the copy
        auto h = upload_f32(b, hv);
        auto s = b.tensor_f32(n, "s");
        bool ok = require(b.add(*s, *h, *delta), "add") && bits_equal(download_f32(b, *s), sum) && bits_equal(download_f32(b, *h), hv);
        // the norm of another tensor comes next: the add runs first, the norm is that tensor's
        auto norm = b.tensor_f32(n, "n");
        ok = ok && require(b.add_n(*s, *h, *delta, n), "add_n") && require(b.rms_norm_batch(*norm, *h, *nw, batch, cols, eps), "norm of h") &&
             bits_equal(download_f32(b, *norm), nplain) && bits_equal(download_f32(b, *s), sum);
        // fewer elements than the norm covers: no fusion, rows past the count keep their values
        auto h2 = upload_f32(b, hv);
        std::vector<float> part = hv;
        for (size_t i = 0; i < n - cols; ++i) part[i] = sum[i];
        std::vector<float> npart(n);
        q8o_rms_norm(part.data(), nwv.data(), npart.data(), batch, cols, cols, cols, eps);
        ok = ok && require(b.add_n(*h2, *h2, *delta, n - cols), "add_n of three rows") &&
             require(b.rms_norm_batch(*norm, *h2, *nw, batch, cols, eps), "norm of four") && bits_equal(download_f32(b, *h2), part) &&
             bits_equal(download_f32(b, *norm), npart);
        // the norm writes over the addend: separate launches, add first
        auto h3 = upload_f32(b, hv);
        auto d3 = upload_f32(b, dv);
        ok = ok && require(b.add_n(*h3, *h3, *d3, n), "add_n") && require(b.rms_norm_batch(*d3, *h3, *nw, batch, cols, eps), "norm into the addend") &&
             bits_equal(download_f32(b, *h3), sum) && bits_equal(download_f32(b, *d3), nref);
        report("add_held_back_other_calls_next", ok);

        // tensors destroyed while the add is held back
        auto h4 = upload_f32(b, hv);
        auto d4 = upload_f32(b, dv);
        ok = require(b.add_n(*h4, *h4, *d4, n), "add_n");
        d4.reset();                                   // the addend goes: the add runs first
        ok = ok && bits_equal(download_f32(b, *h4), sum);
        auto gone = b.tensor_f32(n, "gone");
        ok = ok && require(b.add(*gone, *h4, *delta), "add into a tensor about to go");
        gone.reset();
        ok = ok && require(b.synchronize(), "sync") && bits_equal(download_f32(b, *h4), sum);
        report("add_held_back_tensors_destroyed", ok);

        // under capture: add + norm + projection as a graph, replays equal the eager run
        auto h5 = upload_f32(b, hv);
        auto out = b.tensor_f32(static_cast<size_t>(batch) * rows, "o");
        auto body = [&]() {
            return b.add_n(*h5, *h5, *delta, n).ok && b.rms_norm_batch(*norm, *h5, *nw, batch, cols, eps).ok &&
                   b.q8_0_matmul(*out, *dw, *norm, batch, cols, rows).ok;
        };
        ok = body() && require(b.synchronize(), "sync");
        const auto eager = download_f32(b, *out);
        ok = ok && bits_equal(download_f32(b, *h5), sum);
        ok = ok && b.begin_capture() && body();
        ok = require(b.end_capture(), "end_capture") && ok;
        for (int rep = 0; rep < 3 && ok; ++rep) {
            ok = require(b.copy_bytes_from_host(*h5, 0, hv.data(), n * 4), "reset h") && require(b.zero_tensor(*out), "zero") &&
                 require(b.replay_graph(), "replay") && require(b.synchronize(), "sync");
            ok = ok && bits_equal(download_f32(b, *out), eager) && bits_equal(download_f32(b, *h5), sum);
        }
        // an add left pending when the capture ends is part of the graph
        ok = ok && b.begin_capture() && b.add_n(*h5, *h5, *delta, n).ok;
        ok = require(b.end_capture(), "end_capture") && ok;
        ok = ok && require(b.copy_bytes_from_host(*h5, 0, hv.data(), n * 4), "reset h") && require(b.replay_graph(), "replay") &&
             bits_equal(download_f32(b, *h5), sum);
        report("add_held_back_under_capture", ok);
    }
}

void case_argmax(qw3::HipQ8Backend &b) {
    std::string d;
    const uint32_t n = 248320;
    auto logits = normal_vec(n, 71);
    logits[777] = logits[200000] = 9.5f;   // a tie: the lower index wins
    auto dl = upload_f32(b, logits);
    const q8o_argmax_pair want = q8o_argmax_row(logits.data(), n);
    const qw3::DeviceArgmax got = b.argmax(*dl);
    report("argmax_vocab", got.token == want.index && got.logit == want.value && got.token == 777);

    bool ok = require(b.argmax_launch(*dl), "argmax_launch");
    const qw3::DeviceArgmax late = b.argmax_collect();
    report("argmax_launch_collect", ok && late.token == want.index && late.logit == want.value);

    auto buf = b.argmax_buffer(4);
    ok = buf != nullptr && require(b.argmax_to_buffer(*dl, *buf, 2), "argmax_to_buffer");
    qw3::DeviceArgmax host[4] = {};
    ok = ok && require(b.copy_argmax_buffer_to_host(*buf, host, 3), "copy_argmax_buffer_to_host");
    ok = ok && host[2].token == want.index && host[2].logit == want.value;
    ok = ok && !b.argmax_to_buffer(*dl, *buf, 4).ok && b.argmax_buffer(0) == nullptr;
    report("argmax_to_buffer", ok);

    for (uint32_t stride : {1000u, 50000u, 262144u, 262145u}) {   // the last takes the host scan
        const uint32_t batch = 5;
        auto x = normal_vec(static_cast<size_t>(batch) * stride, 72 + stride);
        x[static_cast<size_t>(3) * stride + 10] = x[static_cast<size_t>(3) * stride + 900] = 8.0f;
        for (uint32_t c = 0; c < stride; ++c) x[static_cast<size_t>(4) * stride + c] = -INFINITY;
        auto dx = upload_f32(b, x);
        std::vector<qw3::DeviceArgmax> rows;
        ok = require(b.argmax_batch(*dx, batch, stride, rows), "argmax_batch");
        std::vector<q8o_argmax_pair> ref(batch);
        if (q8o_argmax_rows(x.data(), batch, stride, ref.data()) != 0) q8o_argmax_rows_scan(x.data(), batch, stride, ref.data());
        for (uint32_t j = 0; j < batch && ok; ++j)
            if (rows[j].token != ref[j].index || std::memcmp(&rows[j].logit, &ref[j].value, 4) != 0) {
                ok = false;
                d = "row " + std::to_string(j) + " got " + std::to_string(rows[j].token) + " want " + std::to_string(ref[j].index);
            }
        report(("argmax_batch_stride" + std::to_string(stride)).c_str(), ok, d);
    }
}

// Embedding lookup: every output is an exact product, so the comparison is on bits.
void case_get_rows(qw3::HipQ8Backend &b) {
    std::string d;
    const uint32_t rows = 3000, cols = 5120;
    const HostWeight w = make_weight(rows, cols, 91);
    auto weight = b.weight_q8_0(w.gguf.data(), rows, cols, "embed");
    auto want_row = [&](uint64_t r) {
        std::vector<float> v(cols);
        q8o_get_row(w.split.data(), r, cols, v.data());
        return v;
    };
    auto same_bits = [](const std::vector<float> &a, const float *ref, size_t n) {
        return std::memcmp(a.data(), ref, n * 4) == 0;
    };

    auto out = b.tensor_f32(cols, "row");
    bool ok = weight != nullptr;
    for (uint64_t r : {0ull, 1234ull, 2999ull}) {
        ok = ok && require(b.q8_0_get_row(*out, *weight, r), "get_row");
        ok = ok && same_bits(download_f32(b, *out), want_row(r).data(), cols);
    }
    ok = ok && !b.q8_0_get_row(*out, *weight, rows).ok;
    report("get_row_f32", ok);

    auto outb = b.tensor_bf16(cols, "rowb");
    ok = require(b.q8_0_get_row(*outb, *weight, 77), "get_row bf16");
    {
        std::vector<uint16_t> raw(cols);
        ok = ok && require(b.copy_bytes_to_host(*outb, raw.data(), 0, cols * 2), "download bf16");
        const auto ref = want_row(77);
        for (uint32_t i = 0; i < cols && ok; ++i) ok = raw[i] == q8o_f32_to_bf16(ref[i]);
    }
    report("get_row_bf16", ok);

    // chained to an argmax slot: the token of a logits row picks the embedding row
    auto logits = normal_vec(rows, 92);
    logits[2024] = 50.0f;
    auto dl = upload_f32(b, logits);
    auto buf = b.argmax_buffer(3);
    ok = buf != nullptr && require(b.argmax_to_buffer(*dl, *buf, 1), "argmax_to_buffer");
    ok = ok && require(b.q8_0_get_row_from_argmax(*out, *weight, *buf, 1), "get_row_from_argmax");
    ok = ok && same_bits(download_f32(b, *out), want_row(2024).data(), cols);
    report("get_row_from_argmax", ok);

    // a slot without a token (all logits -inf -> index -1) gives zeros
    std::vector<float> none(rows, -INFINITY);
    auto dn = upload_f32(b, none);
    ok = require(b.argmax_to_buffer(*dn, *buf, 2), "argmax_to_buffer none");
    ok = ok && require(b.q8_0_get_row_from_argmax(*out, *weight, *buf, 2), "get_row_from_argmax none");
    {
        const auto got = download_f32(b, *out);
        for (uint32_t i = 0; i < cols && ok; ++i) ok = got[i] == 0.0f && !std::signbit(got[i]);
    }
    ok = ok && !b.q8_0_get_row_from_argmax(*out, *weight, *buf, 3).ok;
    report("get_row_from_argmax_no_token", ok);

    const std::vector<uint64_t> ids = {5, 2999, 0, 5, 1500, 42, 2998};
    const uint32_t batch = static_cast<uint32_t>(ids.size());
    auto many = b.tensor_f32(static_cast<size_t>(batch) * cols, "rows");
    ok = require(b.q8_0_get_rows_batch(*many, *weight, ids.data(), batch), "get_rows_batch");
    {
        const auto got = download_f32(b, *many);
        for (uint32_t j = 0; j < batch && ok; ++j)
            ok = std::memcmp(got.data() + static_cast<size_t>(j) * cols, want_row(ids[j]).data(), cols * 4) == 0;
    }
    ok = ok && b.q8_0_get_rows_batch(*many, *weight, ids.data(), 0).ok;
    report("get_rows_batch", ok);
}

// A Q8_0 tensor travels file -> GgufFile -> split-plane device weight -> GEMV and must give what
// the same blocks give when handed to weight_q8_0 directly.
void case_gguf(qw3::HipQ8Backend &b) {
    std::string d;
    const uint32_t rows = 640, cols = 1024;
    const HostWeight w = make_weight(rows, cols, 301);
    const std::string path = "/tmp/q8mi_backend_parity_" + std::to_string(static_cast<long>(getpid())) + ".gguf";
    {
        std::vector<uint8_t> f;
        auto put = [&](const void *p, size_t n) { f.insert(f.end(), static_cast<const uint8_t *>(p), static_cast<const uint8_t *>(p) + n); };
        auto u32 = [&](uint32_t v) { put(&v, 4); };
        auto u64 = [&](uint64_t v) { put(&v, 8); };
        auto str = [&](const char *t) { u64(std::strlen(t)); put(t, std::strlen(t)); };
        put("GGUF", 4); u32(3); u64(2); u64(1);
        str("general.architecture"); u32(8); str("qwen3");
        str("pad.bias"); u32(1); u64(5); u32(0); u64(0);                 // 20 bytes of F32 first, so the weight is not at offset 0
        str("blk.0.attn_output.weight"); u32(2); u64(cols); u64(rows); u32(8); u64(32);
        while (f.size() % 32) f.push_back(0);
        const float bias[5] = {1, 2, 3, 4, 5};
        put(bias, 20);
        while (f.size() % 32) f.push_back(0);
        put(w.gguf.data(), w.gguf.size());
        FILE *fp = std::fopen(path.c_str(), "wb");
        if (fp) { std::fwrite(f.data(), 1, f.size(), fp); std::fclose(fp); }
    }
    bool ok = true;
    try {
        const qw3::GgufFile file(path);
        const qw3::GgufTensorInfo *t = file.find_tensor("blk.0.attn_output.weight");
        ok = t != nullptr && t->type == 8 && qw3::gguf_tensor_rows(*t) == rows && qw3::gguf_tensor_cols(*t) == cols &&
             t->bytes == w.gguf.size() && std::memcmp(file.data() + t->abs_offset, w.gguf.data(), t->bytes) == 0;
        ok = ok && qw3::gguf_upload_q8_0(b, file, "pad.bias") == nullptr && qw3::gguf_upload_q8_0(b, file, "absent") == nullptr;
        auto from_file = qw3::gguf_upload_q8_0(b, file, "blk.0.attn_output.weight");
        auto direct = b.weight_q8_0(w.gguf.data(), rows, cols, "direct");
        ok = ok && from_file != nullptr && direct != nullptr && from_file->rows == rows && from_file->cols == cols;
        const auto x = normal_vec(cols, 302);
        auto dx = upload_f32(b, x);
        auto o1 = b.tensor_f32(rows, "o1"), o2 = b.tensor_f32(rows, "o2");
        ok = ok && require(b.q8_0_matvec(*o1, *from_file, *dx), "matvec gguf") && require(b.q8_0_matvec(*o2, *direct, *dx), "matvec direct");
        std::vector<float> ref, mag;
        oracle_linear(w, x.data(), 1, cols, rows, ref, mag);
        const auto g1 = download_f32(b, *o1);
        ok = ok && g1 == download_f32(b, *o2) && close_fp32(g1, ref, mag, 1, rows, rows, d);
    } catch (const std::exception &e) {
        ok = false;
        d = e.what();
    }
    std::remove(path.c_str());
    report("gguf_tensor_to_matvec", ok, d);
}

void case_lm_head_verify(qw3::HipQ8Backend &b) {
    const uint32_t vocab = 30000, cols = 1024, eos = 5;
    const HostWeight w = make_weight(vocab, cols, 81);
    auto dw = b.weight_q8_0(w.gguf.data(), vocab, cols, "lm");
    for (uint32_t batch : {1u, 4u, 8u}) {
        const auto x = normal_vec(static_cast<size_t>(batch) * cols, 82 + batch);
        auto dx = upload_f32(b, x);
        std::vector<float> ref, mag;
        oracle_linear(w, x.data(), batch, cols, vocab, ref, mag);
        std::vector<q8o_argmax_pair> rows(batch);
        q8o_argmax_rows_scan(ref.data(), batch, vocab, rows.data());
        std::vector<int32_t> toks(batch);
        for (uint32_t j = 0; j < batch; ++j) toks[j] = rows[j].index;
        bool ok = true;
        std::string d;
        for (uint32_t prefix = 0; prefix < batch && ok; ++prefix) {
            std::vector<int32_t> drafts(batch - 1);
            for (uint32_t i = 0; i + 1 < batch; ++i) drafts[i] = i < prefix ? toks[i] : (toks[i] + 1) % static_cast<int32_t>(vocab);
            int32_t want_next = -1;
            const uint32_t want_acc = q8o_accept(toks.data(), drafts.data(), batch - 1, eos, &want_next);
            std::vector<qw3::DeviceArgmax> got;
            uint32_t acc = 99;
            int32_t next = -1;
            ok = require(b.lm_head_verify(*dw, *dx, batch, cols, drafts.data(), batch - 1, eos, got, acc, next), "lm_head_verify");
            ok = ok && acc == want_acc && next == want_next && want_acc == prefix;
            for (uint32_t j = 0; j < batch && ok; ++j) {
                const float tol = 1e-5f * std::fabs(rows[j].value) + 1e-6f * mag[static_cast<size_t>(j) * vocab + rows[j].index];
                ok = got[j].token == rows[j].index && std::fabs(got[j].logit - rows[j].value) <= tol;
            }
            if (!ok) d = "prefix " + std::to_string(prefix);
        }
        // the unfused route through the same API gives the same tokens
        auto logits = b.tensor_f32(static_cast<size_t>(batch) * vocab, "logits");
        std::vector<qw3::DeviceArgmax> unfused;
        ok = ok && require(b.q8_0_matmul(*logits, *dw, *dx, batch, cols, vocab), "lm matmul");
        ok = ok && require(b.argmax_batch(*logits, batch, vocab, unfused), "lm argmax_batch");
        for (uint32_t j = 0; j < batch && ok; ++j) ok = unfused[j].token == rows[j].index;
        report(("lm_head_verify_batch" + std::to_string(batch)).c_str(), ok, d);
    }
}

// A captured decode-style sequence replayed several times with eager work and
// synchronizations in between; every replay must equal the eager result bit for bit.
// rms_norm, rms_norm_batch and rms_norm_q8_0_matmul_fanout at batch 1 (one launch), 3 (fused
// norm + quantizer) and 20 (the two-step base behaviour), with five weights so that a second
// group of the fan-out runs too.  The normalised rows must be the oracle's bits.
void case_rms_norm(qw3::HipQ8Backend &b) {
    const uint32_t cols = 2048;
    const float eps = 1e-6f;
    const uint32_t heights[5] = {768, 130, 31, 256, 64};
    std::vector<HostWeight> hw;
    std::vector<std::unique_ptr<qw3::DeviceWeight>> dw;
    for (int i = 0; i < 5; ++i) {
        hw.push_back(make_weight(heights[i], cols, 300 + i));
        dw.push_back(b.weight_q8_0(hw.back().gguf.data(), heights[i], cols, "w"));
    }
    auto nwv = normal_vec(cols, 310, 0.5f);
    for (auto &f : nwv) f += 1.0f;
    auto nw = b.weight_f32(nwv.data(), cols, "norm.weight");
    std::string d;
    for (uint32_t batch : {1u, 3u, 20u}) {
        const auto x = normal_vec(static_cast<size_t>(batch) * cols, 320 + batch, 3.0f);
        auto dx = upload_f32(b, x);
        std::vector<float> nref(x.size());
        q8o_rms_norm(x.data(), nwv.data(), nref.data(), batch, cols, cols, cols, eps);

        auto plain = b.tensor_f32(x.size(), "plain");
        bool ok = batch == 1 ? require(b.rms_norm(*plain, *dx, *nw, eps), "rms_norm")
                             : require(b.rms_norm_batch(*plain, *dx, *nw, batch, cols, eps), "rms_norm_batch");
        ok = ok && std::memcmp(download_f32(b, *plain).data(), nref.data(), nref.size() * 4) == 0;
        report(("rms_norm_bits_batch" + std::to_string(batch)).c_str(), ok);

        auto normalized = b.tensor_f32(x.size(), "normalized");
        std::vector<std::unique_ptr<qw3::DeviceTensor>> outs;
        qw3::DeviceTensor *op[5];
        const qw3::DeviceWeight *wp[5];
        uint32_t strides[5];
        for (int i = 0; i < 5; ++i) {
            strides[i] = heights[i] + (batch > 1 ? 8 : 0);
            outs.push_back(b.tensor_f32(static_cast<size_t>(batch) * strides[i], "o"));
            op[i] = outs.back().get();
            wp[i] = dw[i].get();
        }
        ok = require(b.rms_norm_q8_0_matmul_fanout(*normalized, op, wp, strides, 5, *dx, *nw, batch, cols, eps), "fanout");
        ok = ok && std::memcmp(download_f32(b, *normalized).data(), nref.data(), nref.size() * 4) == 0;
        if (!ok && d.empty()) d = "normalized rows differ from the oracle";
        for (int i = 0; i < 5 && ok; ++i) {
            std::vector<float> ref, mag;
            if (batch <= 8) {
                oracle_linear(hw[i], nref.data(), batch, cols, strides[i], ref, mag);
                ok = close_fp32(download_f32(b, *op[i]), ref, mag, batch, heights[i], strides[i], d);
            } else {   // above 8 rows the matmul route quantizes to D4 blocks where the shape allows
                auto two = b.tensor_f32(static_cast<size_t>(batch) * strides[i], "two");
                ok = require(b.q8_0_matmul(*two, *dw[i], *plain, batch, cols, strides[i]), "matmul");
                const auto a = download_f32(b, *op[i]), c = download_f32(b, *two);
                for (uint32_t j = 0; j < batch && ok; ++j)
                    ok = std::memcmp(&a[static_cast<size_t>(j) * strides[i]], &c[static_cast<size_t>(j) * strides[i]],
                                     heights[i] * 4) == 0;
                if (!ok) d = "differs from rms_norm_batch + q8_0_matmul";
            }
        }
        report(("rms_norm_q8_0_matmul_fanout_batch" + std::to_string(batch)).c_str(), ok, d);
    }
    // the twins forward to the same operator
    {
        const auto x = normal_vec(cols, 399, 2.0f);
        auto dx = upload_f32(b, x);
        auto n1 = b.tensor_f32(cols, "n1"), n2 = b.tensor_f32(cols, "n2");
        auto o1 = b.tensor_f32(heights[0], "o1"), o2 = b.tensor_f32(heights[0], "o2");
        qw3::DeviceTensor *p1[1] = {o1.get()}, *p2[1] = {o2.get()};
        const qw3::DeviceWeight *wp[1] = {dw[0].get()};
        const uint32_t st[1] = {heights[0]};
        bool ok = require(b.rms_norm_q8_0_matmul_attention_fanout(*n1, p1, wp, st, 1, *dx, *nw, 1, cols, eps), "attention") &&
                  require(b.rms_norm_q8_0_matmul_recurrent_fanout(*n2, p2, wp, st, 1, *dx, *nw, 1, cols, eps), "recurrent");
        ok = ok && download_f32(b, *o1) == download_f32(b, *o2) && download_f32(b, *n1) == download_f32(b, *n2);
        report("rms_norm_fanout_twins", ok);
    }
}

void case_graph_replay(qw3::HipQ8Backend &b) {
    const uint32_t hidden = 1024, ffn = 3072;
    const HostWeight wg = make_weight(ffn, hidden, 91), wu = make_weight(ffn, hidden, 92), wd = make_weight(hidden, ffn, 93);
    auto dg = b.weight_q8_0(wg.gguf.data(), ffn, hidden, "g");
    auto du = b.weight_q8_0(wu.gguf.data(), ffn, hidden, "u");
    auto dd = b.weight_q8_0(wd.gguf.data(), hidden, ffn, "d");
    const auto x0 = normal_vec(hidden, 94);
    auto x = upload_f32(b, x0);
    auto act = b.tensor_f32(ffn, "act");
    auto resid = b.tensor_f32(hidden, "resid");
    auto step = [&]() {
        return b.q8_0_matvec_silu_mul(*act, *dg, *du, *x).ok && b.q8_0_matvec_add(*resid, *dd, *act).ok;
    };
    bool ok = require(b.zero_tensor(*resid), "zero") && step() && require(b.synchronize(), "sync");   // eager: sizes the scratch
    const auto eager = download_f32(b, *resid);
    ok = ok && b.begin_capture() && step();
    ok = require(b.end_capture(), "end_capture") && ok;
    std::string d;
    for (int rep = 0; rep < 4 && ok; ++rep) {
        ok = require(b.zero_tensor(*resid), "zero") && require(b.replay_graph(), "replay") && require(b.synchronize(), "sync");
        const auto got = download_f32(b, *resid);
        if (std::memcmp(got.data(), eager.data(), got.size() * 4) != 0) { ok = false; d = "replay " + std::to_string(rep) + " differs"; }
        // unrelated eager work between replays, using the same scratch
        auto tmp = b.tensor_f32(ffn, "tmp");
        ok = ok && b.q8_0_matvec(*tmp, *dg, *x).ok && require(b.synchronize(), "sync");
    }
    report("graph_replay_x4", ok, d);

    // the fused norm + fan-out (one launch) and a medium-batch matmul (ring-staged tiles), captured
    // together after one eager run and replayed with eager work in between
    {
        const uint32_t mb = 40;
        auto nwv = normal_vec(hidden, 97, 0.3f);
        for (auto &f : nwv) f += 1.0f;
        auto nw = b.weight_f32(nwv.data(), hidden, "norm.weight");
        auto normalized = b.tensor_f32(hidden, "normalized");
        auto fo = b.tensor_f32(ffn, "fo");
        qw3::DeviceTensor *outs[1] = {fo.get()};
        const qw3::DeviceWeight *ws[1] = {dg.get()};
        const uint32_t strides[1] = {ffn};
        auto xm = upload_f32(b, normal_vec(static_cast<size_t>(mb) * hidden, 98));
        auto om = b.tensor_f32(static_cast<size_t>(mb) * ffn, "om");
        auto step2 = [&]() {
            return b.rms_norm_q8_0_matmul_fanout(*normalized, outs, ws, strides, 1, *x, *nw, 1, hidden, 1e-6f).ok &&
                   b.q8_0_matmul(*om, *du, *xm, mb, hidden, ffn).ok;
        };
        bool ok2 = step2() && require(b.synchronize(), "sync");
        const auto e1 = download_f32(b, *fo), e2 = download_f32(b, *om);
        ok2 = ok2 && b.begin_capture() && step2();
        ok2 = require(b.end_capture(), "end_capture") && ok2;
        std::string d2;
        for (int rep = 0; rep < 3 && ok2; ++rep) {
            ok2 = require(b.zero_tensor(*fo), "zero") && require(b.zero_tensor(*om), "zero") &&
                  require(b.replay_graph(), "replay") && require(b.synchronize(), "sync");
            const auto g1 = download_f32(b, *fo), g2 = download_f32(b, *om);
            if (std::memcmp(g1.data(), e1.data(), g1.size() * 4) != 0 || std::memcmp(g2.data(), e2.data(), g2.size() * 4) != 0) {
                ok2 = false;
                d2 = "replay " + std::to_string(rep) + " differs";
            }
            auto tmp = b.tensor_f32(ffn, "tmp");
            ok2 = ok2 && b.q8_0_matvec(*tmp, *dg, *x).ok && require(b.synchronize(), "sync");
        }
        report("graph_replay_norm_fanout_and_medium_matmul", ok2, d2);
    }

    // growth of a scratch buffer is refused while capturing
    const HostWeight wbig = make_weight(64, 8192, 95);
    auto dbig = b.weight_q8_0(wbig.gguf.data(), 64, 8192, "big");
    auto xbig = upload_f32(b, normal_vec(static_cast<size_t>(8) * 8192, 96));
    auto obig = b.tensor_f32(8 * 64, "obig");
    ok = b.begin_capture();
    const bool refused = !b.q8_0_matmul(*obig, *dbig, *xbig, 8, 8192, 64).ok;
    (void)b.end_capture();
    report("capture_refuses_scratch_growth", ok && refused);
}

}  // namespace

int main(int argc, char **argv) {
    const std::string only = argc > 1 ? argv[1] : "";
    qw3::HipQ8Backend backend;
    std::printf("backend: %s\n", backend.name());
    struct Case { const char *name; void (*fn)(qw3::HipQ8Backend &); };
    const Case cases[] = {
        {"closed_form", case_closed_form}, {"matvec", case_matvec_family}, {"matmul", case_matmul},
        {"matmul_add", case_matmul_add_batched}, {"silu_mul", case_silu_mul}, {"norm_reuse", case_norm_reuse}, {"add_held_back", case_add_held_back},
        {"argmax", case_argmax}, {"get_rows", case_get_rows}, {"gguf", case_gguf}, {"lm_head", case_lm_head_verify}, {"rms_norm", case_rms_norm}, {"graph", case_graph_replay},
    };
    for (const auto &c : cases) {
        if (!only.empty() && only != c.name) continue;
        std::printf("== %s\n", c.name);
        std::fflush(stdout);
        c.fn(backend);
    }
    require(backend.end(), "end");
    std::printf("%d cases, %d failed\n", g_cases, g_failed);
    return g_failed == 0 && g_cases > 0 ? 0 : 1;
}

// Exercises the C++ host mirror (vtl_amd/host/vtl_hip.hpp) against the CPU
// oracle on a real device: alloc -> H2D -> op -> D2H -> release, plus the error
// paths.  Links libvtlhip.so (product) and libvtloracle.so (checker).
// Exit code 0 = all checks passed.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>

#include "vtl_hip.hpp"
#include "vtl_oracle.h"

static int failures = 0;
#define CHECK(cond)                                                        \
    do {                                                                   \
        if (!(cond)) {                                                     \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);    \
            failures++;                                                    \
        }                                                                  \
    } while (0)

int main(int argc, char **argv)
{
    const bool no_device = argc > 1 && !std::strcmp(argv[1], "--no-device");
    // error paths that need no device
    CHECK(vtl_hip_quantize_f32_i8(nullptr, 1, 1, 1, nullptr, nullptr) == VTL_HIP_ERR_INVALID_ARG);
    CHECK(vtl_hip_free(nullptr) == VTL_HIP_OK);
    try {
        vtl::per_row_of(3);
        CHECK(false);
    } catch (const std::invalid_argument &) {
    }
    try {
        int m, n, k;
        vtl::matmul_shapes({4, 32}, {6, 48}, m, n, k);
        CHECK(false);
    } catch (const std::invalid_argument &e) {
        CHECK(std::strstr(e.what(), "Invalid shapes for matrix multiplication"));
    }
    if (no_device) {
        std::printf(failures ? "host mirror: %d failure(s)\n" : "host mirror (no device): ok\n", failures);
        return failures ? 1 : 0;
    }

    int ndev = 0;
    CHECK(vtl_hip_device_count(&ndev) == VTL_HIP_OK && ndev > 0);
    if (ndev <= 0)
        return 1;
    try {
        vtl::HipStorage<float> bad(4, vtl::HipParams{ndev + 7});
        CHECK(false);
    } catch (const vtl::HipError &e) {
        CHECK(e.status == VTL_HIP_ERR_NO_DEVICE);
    }

    std::mt19937 rng(1234);
    std::normal_distribution<float> nd(0.f, 1.f);
    const int M = 37, K = 256, N = 96;
    std::vector<float> x((size_t)M * K), w((size_t)N * K), b(N);
    for (auto &v : x) v = nd(rng);
    for (auto &v : w) v = nd(rng) * 0.02f;
    for (auto &v : b) v = nd(rng) * 0.1f;

    // storage round trip
    auto st = vtl::HipStorage<float>::from_cpu(x);
    CHECK(st.count == x.size() && st.size == x.size() * 4);
    CHECK(st.to_array() == x);
    st.release();
    CHECK(st.ptr == nullptr);

    // quantize / dequantize vs oracle
    auto xt = vtl::HipTensor<float>::from_host(x, {M, K});
    CHECK(xt.is_matrix() && xt.strides == (std::vector<int>{K, 1}) && xt.numel() == (size_t)M * K);
    for (int axis : {0, -1}) {
        auto qs = vtl::quantize_i8(xt, axis);
        std::vector<int8_t> qr(x.size());
        std::vector<float> sr(axis == 0 ? M : 1);
        vtl_ref_quantize_f32_i8(x.data(), M, K, axis == 0, qr.data(), sr.data());
        CHECK(qs.first.cpu() == qr);
        CHECK(qs.second.cpu() == sr);
        auto d = vtl::dequantize(qs.first, qs.second, axis);
        std::vector<float> dr(x.size());
        vtl_ref_dequantize_i8_f32(qr.data(), sr.data(), M, K, axis == 0, dr.data());
        CHECK(d.cpu() == dr);
    }

    // int8 gemm vs oracle
    {
        std::vector<int8_t> a((size_t)M * K), bt((size_t)N * K);
        std::uniform_int_distribution<int> ud(-127, 127);
        for (auto &v : a) v = (int8_t)ud(rng);
        for (auto &v : bt) v = (int8_t)ud(rng);
        auto A = vtl::HipTensor<int8_t>::from_host(a, {M, K});
        auto B = vtl::HipTensor<int8_t>::from_host(bt, {N, K});
        vtl::HipTensor<int32_t> C({M, N});
        vtl::gemm_i8_hip(C, A, B);
        std::vector<int32_t> ref((size_t)M * N);
        vtl_ref_gemm_i8_i32(a.data(), bt.data(), ref.data(), M, N, K, 1);
        CHECK(C.cpu() == ref);
        vtl::HipTensor<int32_t> wrong({M, N + 1});
        try {
            vtl::gemm_i8_hip(wrong, A, B);
            CHECK(false);
        } catch (const std::invalid_argument &) {
        }
    }

    // the Linear hook vs oracle (per-output-channel weights, per-token activations)
    {
        auto y = vtl::linear_forward_hip_f32(x, M, K, w, N, &b, true);
        std::vector<int8_t> wq(w.size());
        std::vector<float> sw(N), ref((size_t)M * N);
        vtl_ref_quantize_f32_i8(w.data(), N, K, 1, wq.data(), sw.data());
        vtl_ref_linear_f32_dynquant(x.data(), wq.data(), sw.data(), b.data(), ref.data(), M, N, K, 1, 1);
        CHECK(y == ref);
        try {
            vtl::linear_forward_hip_f32(x, M, K + 1, w, N, &b);
            CHECK(false);
        } catch (const std::invalid_argument &) {
        }
    }
    // the session: weights quantized once and kept on the device, staging buffer reused,
    // activations handed from layer to layer (autograd_hip/hip_session_d_hip.v)
    {
        const int H = 64, O = 24;
        std::vector<float> w2((size_t)O * N), b2(O), w1b = w;
        for (auto &v : w2) v = nd(rng) * 0.05f;
        for (auto &v : b2) v = nd(rng) * 0.1f;
        (void)H;
        vtl::HipSession s;
        s.init_device();
        CHECK(s.enabled);
        auto ref_linear = [&](const std::vector<float> &xin, int m, int k, const std::vector<float> &wf, int n,
                              const std::vector<float> &bf, bool relu) {
            std::vector<int8_t> wq(wf.size());
            std::vector<float> sw(n), out((size_t)m * n);
            vtl_ref_quantize_f32_i8(wf.data(), n, k, 1, wq.data(), sw.data());
            vtl_ref_linear_f32_dynquant(xin.data(), wq.data(), sw.data(), bf.data(), out.data(), m, n, k, relu, 1);
            return out;
        };
        // frozen parameters (inference): quantized once, the copy is kept
        auto y1 = s.linear_forward_f32(x, M, K, w, N, b, &w, nullptr, true);
        void *ws_first = s.workspace.ptr;
        void *codes_first = s.layers[0].w_q.data.ptr;
        auto y1b = s.linear_forward_f32(x, M, K, w, N, b, &w, nullptr, true);
        CHECK(s.layers.size() == 1 && s.quantize_count == 1);          // quantized once
        CHECK(s.workspace.ptr == ws_first && s.layers[0].w_q.data.ptr == codes_first);
        CHECK(y1 == y1b && y1 == ref_linear(x, M, K, w, N, b, false));
        // Adam assigns a new weight tensor: same slot, new codes
        for (auto &v : w1b) v = -v;
        auto y1c = s.linear_forward_f32(x, M, K, w1b, N, b, &w, nullptr, true);
        CHECK(s.layers.size() == 1 && s.quantize_count == 2);
        CHECK(y1c == ref_linear(x, M, K, w1b, N, b, false));
        // SGD-style step: the SAME tensor updated in place (nn/internal/optimizers.v:6-12).  A
        // training forward (not frozen) quantizes every time and always sees the new values ...
        {
            std::vector<float> wt = w, bt = b;
            const int before = s.quantize_count;
            auto t0 = s.linear_forward_f32(x, M, K, wt, N, bt, &wt, nullptr);
            CHECK(t0 == ref_linear(x, M, K, wt, N, bt, false));
            for (size_t i = 0; i < wt.size(); i++) wt[i] -= 0.1f * w1b[i];
            for (auto &v : bt) v -= 0.05f;
            auto t1 = s.linear_forward_f32(x, M, K, wt, N, bt, &wt, nullptr);
            CHECK(t1 == ref_linear(x, M, K, wt, N, bt, false));
            CHECK(s.quantize_count == before + 2);
            // ... a frozen forward does not trust the copy a training forward made ...
            for (size_t i = 0; i < wt.size(); i++) wt[i] += 0.3f * w1b[i];
            auto t2 = s.linear_forward_f32(x, M, K, wt, N, bt, &wt, nullptr, true);
            CHECK(t2 == ref_linear(x, M, K, wt, N, bt, false) && s.quantize_count == before + 3);
            auto t3 = s.linear_forward_f32(x, M, K, wt, N, bt, &wt, nullptr, true);
            CHECK(t3 == t2 && s.quantize_count == before + 3);
            // ... and notices an in-place edit of frozen parameters by their fingerprint
            for (auto &v : wt) v *= 0.5f;
            auto t4 = s.linear_forward_f32(x, M, K, wt, N, bt, &wt, nullptr, true);
            CHECK(t4 == ref_linear(x, M, K, wt, N, bt, false) && s.quantize_count == before + 4);
            for (auto &v : bt) v = 0.25f;
            auto t5 = s.linear_forward_f32(x, M, K, wt, N, bt, &wt, nullptr, true);
            CHECK(t5 == ref_linear(x, M, K, wt, N, bt, false));
            s.invalidate(&wt);
            auto t6 = s.linear_forward_f32(x, M, K, wt, N, bt, &wt, nullptr, true);
            CHECK(t6 == t5 && s.quantize_count == before + 5);
        }
        // Linear -> ReLU -> Linear with the activation staying on the device
        auto h = s.linear_forward_f32(x, M, K, w, N, b, &w, nullptr);
        CHECK(s.has_pending);
        auto h_dev = s.take_pending();
        auto r = s.relu_forward_f32(std::move(h_dev));
        std::vector<float> r_ref = h;
        vtl_ref_relu_f32(r_ref.data(), (int64_t)r_ref.size());
        CHECK(r == r_ref);
        auto r_dev = s.take_pending();
        auto out = s.linear_forward_f32(r, M, N, w2, O, b2, &w2, &r_dev);
        CHECK(out == ref_linear(r_ref, M, N, w2, O, b2, false));
        CHECK(s.layers.size() == 3);
        // the whole chain with int8 hand-off equals the layer-by-layer result bit for bit
        auto chain = s.mlp_forward_i8(x, M, {&w, &w2}, {&b, &b2}, {K, N, O}, {true, false});
        auto h_relu = ref_linear(x, M, K, w, N, b, true);
        CHECK(chain == ref_linear(h_relu, M, N, w2, O, b2, false));
        // a few tokens take the route on which every layer quantizes its own input: same bits
        for (int few : {1, 5, 32}) {
            std::vector<float> xf(x.begin(), x.begin() + (size_t)few * K);
            auto got = s.mlp_forward_i8(xf, few, {&w, &w2}, {&b, &b2}, {K, N, O}, {true, false});
            auto hf = ref_linear(xf, few, K, w, N, b, true);
            CHECK(got == ref_linear(hf, few, N, w2, O, b2, false));
        }
        s.release();
    }
    // la.matmul and LinearGate.backward with f64 accumulation vs oracle: integer-valued
    // operands, for which every summation order gives the same bits
    {
        std::uniform_int_distribution<int> ud(-8, 8);
        std::vector<float> g((size_t)M * N), xi((size_t)M * K), wi((size_t)N * K);
        for (auto &v : g) v = (float)ud(rng);
        for (auto &v : xi) v = (float)ud(rng);
        for (auto &v : wi) v = (float)ud(rng);
        auto G = vtl::HipTensor<float>::from_host(g, {M, N});
        auto W = vtl::HipTensor<float>::from_host(wi, {N, K});
        auto X = vtl::HipTensor<float>::from_host(xi, {M, K});
        std::vector<float> ref((size_t)M * K);
        vtl_ref_matmul_f32(g.data(), wi.data(), ref.data(), M, K, N, 0, 0, 1);
        CHECK(vtl::matmul_hip(G, W).cpu() == ref);                 // grad . W
        std::vector<float> ref_t((size_t)N * K);
        vtl_ref_matmul_f32(g.data(), xi.data(), ref_t.data(), N, K, M, 1, 0, 1);
        CHECK(vtl::matmul_hip(G, X, true, false).cpu() == ref_t);  // grad^T . x
        try {
            vtl::matmul_hip(G, X);
            CHECK(false);
        } catch (const std::invalid_argument &e) {
            CHECK(std::strstr(e.what(), "Invalid shapes for matrix multiplication"));
        }
        std::vector<float> dx((size_t)M * K), dw((size_t)N * K), db(N);
        vtl_ref_linear_backward_f32(g.data(), xi.data(), wi.data(), dx.data(), dw.data(), db.data(), M, N, K, 1);
        auto got = vtl::linear_backward_hip_f32(g, M, N, xi, K, wi, true);
        CHECK(got[0] == dx && got[1] == dw && got[2] == db);
        auto no_bias = vtl::linear_backward_hip_f32(g, M, N, xi, K, wi, false);
        CHECK(no_bias[0] == dx && no_bias[2] == std::vector<float>(N, 0.0f));
    }
    // generic tensor operations vs oracle
    {
        std::uniform_int_distribution<int> ud(-8, 8);
        std::vector<double> a((size_t)M * K), xv(K), yr(M);
        for (auto &v : a) v = ud(rng);
        for (auto &v : xv) v = ud(rng);
        auto A = vtl::HipTensor<double>::from_host(a, {M, K});
        auto X = vtl::HipTensor<double>::from_host(xv, {K});
        vtl::HipTensor<double> Y({M});
        vtl::gemv_hip(Y, A, X);
        vtl_ref_gemv_f64(a.data(), xv.data(), yr.data(), M, K);
        CHECK(Y.cpu() == yr);                       // integer-valued: exact in any order
        try {
            vtl::gemv_hip(Y, A, Y);
            CHECK(false);
        } catch (const std::invalid_argument &) {
        }
        auto R = vtl::HipTensor<float>::from_host(x, {M, K});
        vtl::relu_hip(R);
        std::vector<float> rr = x;
        vtl_ref_relu_f32(rr.data(), (int64_t)rr.size());
        CHECK(R.cpu() == rr);
        auto S = vtl::sigmoid_hip(xt);
        std::vector<float> sr(x.size());
        vtl_ref_sigmoid_f32(x.data(), sr.data(), (int64_t)x.size());
        auto sg = S.cpu();
        int worst = 0;
        for (size_t i = 0; i < sr.size(); i++) {
            int32_t u, v;
            std::memcpy(&u, &sg[i], 4);
            std::memcpy(&v, &sr[i], 4);
            worst = std::max(worst, std::abs(u - v));
        }
        CHECK(worst <= 1);                          // the device's f64 exp against the C library's
    }
    std::printf(failures ? "host mirror: %d failure(s)\n" : "host mirror: ok\n", failures);
    return failures ? 1 : 0;
}

// Testbench-style harness for the host-side module mirror (flexllm_modules.h), shaped like the reference's
// *_tb.cpp files: build seeded inputs in the stream packings, push them through the module functions, compare
// with an in-process golden, print a check mark or a cross.  Unlike the reference's harnesses the exit code is
// non-zero when a check fails.
//
//   QuantWrapper linear, decode   <-> SpinQuant_Llama_32_1B/Linear_Layer_Decoding_tb.cpp:93-251 (1e-2 relative)
//   QuantWrapper linear, prefill  <-> SpinQuant_Llama_32_1B/Linear_Layer_Prefilling_tb.cpp (1e-2 relative)
//   MHA prefill                   <-> SpinQuant_Llama_32_1B/MHA_i8xi8_prefilling_tb.cpp:12-268 (5e-3 relative)
//   FHT / RMSNorm / Swish / residual / softmax against float64 closed forms
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <iostream>
#include <random>
#include <vector>
#include "../flexllm_modules.h"

using namespace fxhost;

constexpr int HIDDEN_DIM = 2048, KV_HIDDEN_DIM = 512, HEAD_DIM = 64, INTER_DIM = 8192;
constexpr int Q_HEAD_NUM = 32, KV_HEAD_NUM = 8;
constexpr int TOKEN_PARALLEL = 8, T_BLOCK_PARALLEL = 8, DEC_W_PARALLEL = 64;

static int failures = 0;
static void verdict(const char* name, bool ok) {
    std::cout << (ok ? "\xE2\x9C\x85 " : "\xE2\x9D\x8C ") << name << (ok ? " passed correctness check!" : " failed!") << std::endl;
    if (!ok) failures++;
}

// symmetric int8 quantisation of a weight matrix per output channel, like the testbenches' w_max/7 with 127
static void quantise_weights(std::vector<float>& w_gold, int n, int k, std::vector<int8_t>& q, std::vector<float>& s) {
    q.resize((size_t)n * k); s.resize(n);
    for (int i = 0; i < n; i++) {
        float w_max = 0;
        for (int j = 0; j < k; j++) w_max = std::max(w_max, std::abs(w_gold[(size_t)i * k + j]));
        float scale = w_max / 127.0f;
        if (scale == 0) scale = 1.0f;
        s[i] = scale;
        for (int j = 0; j < k; j++) {
            int qv = (int)std::round(w_gold[(size_t)i * k + j] / scale);
            qv = std::max(-128, std::min(127, qv));
            q[(size_t)i * k + j] = (int8_t)qv;
            w_gold[(size_t)i * k + j] = qv * scale;
        }
    }
}

static void QuantWrapper_Linear_Layer_q_decoding_test() {
    const int T = 8, K = HIDDEN_DIM, N = HIDDEN_DIM, BP = T_BLOCK_PARALLEL, per = K / BP;
    std::default_random_engine gen(42);
    std::uniform_real_distribution<float> dist(-1.0, 1.0);
    std::vector<float> input_gold((size_t)T * K), weight_gold((size_t)N * K);
    std::vector<vec<float, BP>> input_mmap((size_t)T * per);
    for (int i = 0; i < T; i++) {
        float amax = 0;
        for (int j = 0; j < K; j++) {
            float val = dist(gen);
            input_gold[(size_t)i * K + j] = val;
            amax = std::max(amax, std::abs(val));
            input_mmap[(size_t)i * per + j % per][j / per] = val;            // decode packing
        }
        float scale = amax / 127.0f;
        if (scale == 0) scale = 1.0f;
        for (int j = 0; j < K; j++) input_gold[(size_t)i * K + j] = std::round(input_gold[(size_t)i * K + j] / scale) * scale;   // fake quant
    }
    for (auto& v : weight_gold) v = dist(gen);
    std::vector<int8_t> wq; std::vector<float> ws;
    quantise_weights(weight_gold, N, K, wq, ws);
    DeviceWeight weight(wq.data(), N, K, ws.data());

    std::vector<vec<float, BP>> output_mmap((size_t)T * N / BP);
    for (int t = 0; t < T; t++) {
        stream<vec<float, BP>> x_s, y_s;
        stream<vec<float, 1>> s_b, s_b2, w_s;
        stream<vec<int8_t, BP>> q_s;
        stream<vec<int32_t, BP>> acc_s;
        for (int k = 0; k < per; k++) x_s.write(input_mmap[(size_t)t * per + k]);
        dec_quant_layer_fp32_qint<8, false, BP, HIDDEN_DIM>(x_s, s_b, q_s, K);
        dec_Linear_Layer_i8xi8<BP, DEC_W_PARALLEL, HIDDEN_DIM, 11, HIDDEN_DIM>(q_s, weight, acc_s, K, N);
        // weight scale stream in the order dec_dequant_layer_qint_fp32_bandwidth consumes it (Modules/quant.h:491-501)
        for (int kk = 0; kk < N / (BP * DEC_W_PARALLEL); kk++)
            for (int m = 0; m < BP; m++)
                for (int n = 0; n < DEC_W_PARALLEL; n++) { vec<float, 1> p; p[0] = ws[(size_t)m * (N / BP) + kk * DEC_W_PARALLEL + n]; w_s.write(p); }
        dec_dequant_layer_qint_fp32_bandwidth<8, false, BP, DEC_W_PARALLEL, HIDDEN_DIM>(acc_s, s_b, w_s, y_s, N);
        for (int k = 0; k < N / BP; k++) output_mmap[(size_t)t * (N / BP) + k] = y_s.read();
    }
    bool correct = true;
    for (int i = 0; i < T && correct; i++)
        for (int j = 0; j < N; j++) {
            double gold = 0;
            for (int k = 0; k < K; k++) gold += (double)input_gold[(size_t)i * K + k] * weight_gold[(size_t)j * K + k];
            const float my = output_mmap[(size_t)i * (N / BP) + j % (N / BP)][j / (N / BP)];
            if (std::abs(my - gold) > 1e-2 * std::abs(gold) + 1e-4) { correct = false; std::cout << "Mismatch at (" << i << ", " << j << "): My: " << my << ", Ref_fq: " << gold << std::endl; break; }
        }
    verdict("QuantWrapper Linear Layer (decode, W8A8)", correct);
}

// The reference's own configuration of this testbench (Linear_Layer_Decoding_tb.cpp:93-251): asymmetric uint4
// activations, symmetric int4 weights, dequant with zero point times the row sum of the dequantised weights.
static void QuantWrapper_Linear_Layer_q_decoding_w4a4_test() {
    const int T = 8, K = HIDDEN_DIM, N = HIDDEN_DIM, BP = T_BLOCK_PARALLEL, per = K / BP;
    std::default_random_engine gen(42);
    std::uniform_real_distribution<float> dist(-1.0, 1.0);
    std::vector<float> input_gold((size_t)T * K), weight_gold((size_t)N * K), weight_s(N), weight_sum(N);
    std::vector<int8_t> q_weight((size_t)N * K);
    std::vector<vec<float, BP>> input_mmap((size_t)T * per);
    for (int i = 0; i < T; i++) {
        float vmax = -1e30f, vmin = 1e30f;
        for (int j = 0; j < K; j++) {
            float val = dist(gen);
            input_gold[(size_t)i * K + j] = val;
            vmax = std::max(vmax, val); vmin = std::min(vmin, val);
            input_mmap[(size_t)i * per + j % per][j / per] = val;
        }
        float scale = (vmax - vmin) / 15.0f;
        if (scale == 0) scale = 1.0f;
        for (int j = 0; j < K; j++) {          // fake quant, …_tb.cpp:137-147
            float& v = input_gold[(size_t)i * K + j];
            v = std::round((v - vmin) / scale) * scale + vmin;
        }
    }
    for (int i = 0; i < N; i++) {              // …_tb.cpp:160-190
        float w_max = 0;
        for (int j = 0; j < K; j++) { weight_gold[(size_t)i * K + j] = dist(gen); w_max = std::max(w_max, std::abs(weight_gold[(size_t)i * K + j])); }
        float scale = w_max / 7.0f;
        if (scale == 0) scale = 1.0f;
        weight_s[i] = scale; weight_sum[i] = 0;
        for (int j = 0; j < K; j++) {
            int qval = (int)std::round(weight_gold[(size_t)i * K + j] / scale);
            qval = std::max(-8, std::min(7, qval));
            weight_gold[(size_t)i * K + j] = qval * scale;
            q_weight[(size_t)i * K + j] = (int8_t)qval;
            weight_sum[i] += weight_gold[(size_t)i * K + j];
        }
    }
    DeviceWeight4 weight(q_weight.data(), N, K);
    std::vector<vec<float, BP>> output_mmap((size_t)T * N / BP);
    for (int t = 0; t < T; t++) {
        stream<vec<float, BP>> x_s, y_s;
        stream<vec<float, 2>> s_b, w_s;
        stream<vec<uint8_t, BP>> q_s;
        stream<vec<int32_t, BP>> acc_s;
        for (int k = 0; k < per; k++) x_s.write(input_mmap[(size_t)t * per + k]);
        dec_quant_layer_fp32_qint<4, true, BP, HIDDEN_DIM>(x_s, s_b, q_s, K);
        dec_Linear_Layer_i4xi4<BP, DEC_W_PARALLEL, HIDDEN_DIM, 11, HIDDEN_DIM, true>(q_s, weight, acc_s, K, N);
        for (int kk = 0; kk < N / (BP * DEC_W_PARALLEL); kk++)
            for (int m = 0; m < BP; m++)
                for (int n = 0; n < DEC_W_PARALLEL; n++) {
                    vec<float, 2> p;
                    p[0] = weight_s[(size_t)m * (N / BP) + kk * DEC_W_PARALLEL + n];
                    p[1] = weight_sum[(size_t)m * (N / BP) + kk * DEC_W_PARALLEL + n];
                    w_s.write(p);
                }
        dec_dequant_layer_qint_fp32_bandwidth<4, true, BP, DEC_W_PARALLEL, HIDDEN_DIM>(acc_s, s_b, w_s, y_s, N);
        for (int k = 0; k < N / BP; k++) output_mmap[(size_t)t * (N / BP) + k] = y_s.read();
    }
    bool correct = true;
    for (int i = 0; i < T && correct; i++)
        for (int j = 0; j < N; j++) {
            double gold = 0;
            for (int k = 0; k < K; k++) gold += (double)input_gold[(size_t)i * K + k] * weight_gold[(size_t)j * K + k];
            const float my = output_mmap[(size_t)i * (N / BP) + j % (N / BP)][j / (N / BP)];
            if (std::abs(my - gold) > 1e-2 * std::abs(gold) + 1e-3) { correct = false; std::cout << "Mismatch at (" << i << ", " << j << "): My: " << my << ", Ref_fq: " << gold << std::endl; break; }
        }
    verdict("QuantWrapper Linear Layer (decode, W4A4 asymmetric: the reference's shipped configuration)", correct);
}

static void QuantWrapper_Linear_Layer_q_prefilling_test() {
    const int S = 64, K = HIDDEN_DIM, N = KV_HIDDEN_DIM, TP = TOKEN_PARALLEL;
    std::default_random_engine gen(42);
    std::uniform_real_distribution<float> dist(-1.0, 1.0);
    std::vector<float> input_gold((size_t)S * K), weight_gold((size_t)N * K);
    stream<vec<float, TP>> x_s;
    std::vector<vec<float, TP>> input_mmap((size_t)S / TP * K);
    for (int i = 0; i < S; i++) {
        float amax = 0;
        for (int j = 0; j < K; j++) {
            float val = dist(gen);
            input_gold[(size_t)i * K + j] = val;
            amax = std::max(amax, std::abs(val));
            input_mmap[(size_t)(i / TP) * K + j][i % TP] = val;               // prefill packing
        }
        float scale = amax / 127.0f;
        for (int j = 0; j < K; j++) input_gold[(size_t)i * K + j] = std::round(input_gold[(size_t)i * K + j] / scale) * scale;
    }
    for (auto& v : weight_gold) v = dist(gen);
    std::vector<int8_t> wq; std::vector<float> ws;
    quantise_weights(weight_gold, N, K, wq, ws);
    DeviceWeight weight(wq.data(), N, K, ws.data());
    for (auto& p : input_mmap) x_s.write(p);
    stream<vec<float, 1>> s_b, w_s;
    stream<vec<int8_t, TP>> q_s;
    stream<vec<int32_t, TP>> acc_s;
    stream<vec<float, TP>> y_s;
    pref_quant_layer_fp32_qint<8, false, TP, HIDDEN_DIM>(x_s, s_b, q_s, S, K);
    pref_Linear_Layer_i8xi8<TP, 16, HIDDEN_DIM, 11, KV_HIDDEN_DIM>(q_s, weight, acc_s, S, K, N);
    for (int M = 0; M < S / TP; M++)
        for (int j = 0; j < N; j++) { vec<float, 1> p; p[0] = ws[j]; w_s.write(p); }
    pref_dequant_layer_qint_fp32<8, false, TP, KV_HIDDEN_DIM>(acc_s, s_b, w_s, y_s, S, N);
    std::vector<vec<float, TP>> output_mmap((size_t)S / TP * N);
    for (auto& p : output_mmap) p = y_s.read();
    bool correct = true;
    for (int i = 0; i < S && correct; i++)
        for (int j = 0; j < N; j++) {
            double gold = 0;
            for (int k = 0; k < K; k++) gold += (double)input_gold[(size_t)i * K + k] * weight_gold[(size_t)j * K + k];
            const float my = output_mmap[(size_t)(i / TP) * N + j][i % TP];
            if (std::abs(my - gold) > 1e-2 * std::abs(gold) + 1e-4) { correct = false; std::cout << "Mismatch at (" << i << ", " << j << "): My: " << my << ", Ref_fq: " << gold << std::endl; break; }
        }
    verdict("QuantWrapper Linear Layer (prefill, W8A8)", correct);
}

static void hadamard_gold(std::vector<double>& x) {       // in-place Sylvester transform, natural order
    const size_t n = x.size();
    for (size_t h = 1; h < n; h <<= 1)
        for (size_t i = 0; i < n; i += 2 * h)
            for (size_t j = i; j < i + h; j++) { const double u = x[j], v = x[j + h]; x[j] = u + v; x[j + h] = u - v; }
}

static void FHT_test() {
    const int S = 16, TP = TOKEN_PARALLEL, N = INTER_DIM;
    std::default_random_engine gen(42);
    std::normal_distribution<float> dist(0.0f, 1.0f);
    std::vector<float> x((size_t)S * N);
    for (auto& v : x) v = dist(gen);
    stream<vec<float, TP>> in, out;
    for (int M = 0; M < S / TP; M++)
        for (int k = 0; k < N; k++) { vec<float, TP> p; for (int m = 0; m < TP; m++) p[m] = x[(size_t)(M * TP + m) * N + k]; in.write(p); }
    pref_FHT<float, TP, INTER_DIM, 13>(in, out, S, 90.50966799f);
    std::vector<float> y((size_t)S * N);
    for (int M = 0; M < S / TP; M++)
        for (int k = 0; k < N; k++) { auto p = out.read(); for (int m = 0; m < TP; m++) y[(size_t)(M * TP + m) * N + k] = p[m]; }
    bool correct = true;
    for (int t = 0; t < S; t++) {
        std::vector<double> g(x.begin() + (size_t)t * N, x.begin() + (size_t)(t + 1) * N);
        hadamard_gold(g);
        for (int k = 0; k < N; k++)
            if (std::abs(y[(size_t)t * N + k] - g[k] / 90.50966799) > 2e-5) { correct = false; break; }
    }
    // decode form, block-partitioned lanes
    stream<vec<float, T_BLOCK_PARALLEL>> din, dout;
    const int per = N / T_BLOCK_PARALLEL;
    for (int k = 0; k < per; k++) { vec<float, T_BLOCK_PARALLEL> p; for (int i = 0; i < T_BLOCK_PARALLEL; i++) p[i] = x[(size_t)i * per + k]; din.write(p); }
    dec_FHT<float, T_BLOCK_PARALLEL, INTER_DIM, 13>(din, dout, 90.50966799f);
    for (int k = 0; k < per; k++) { auto p = dout.read(); for (int i = 0; i < T_BLOCK_PARALLEL; i++) if (p[i] != y[(size_t)i * per + k]) correct = false; }
    verdict("FHT R4 (prefill and decode streams, n=8192)", correct);
}

static void Elementwise_test() {
    const int S = 16, TP = TOKEN_PARALLEL, H = HIDDEN_DIM;
    std::default_random_engine gen(7);
    std::normal_distribution<float> dist(0.0f, 2.0f);
    std::vector<float> x((size_t)S * H), r((size_t)S * H), gamma(H);
    for (auto& v : x) v = dist(gen);
    for (auto& v : r) v = dist(gen);
    for (auto& v : gamma) v = 0.5f + std::abs(dist(gen)) * 0.25f;
    auto push = [&](stream<vec<float, TP>>& s, const std::vector<float>& a) {
        for (int M = 0; M < S / TP; M++)
            for (int k = 0; k < H; k++) { vec<float, TP> p; for (int m = 0; m < TP; m++) p[m] = a[(size_t)(M * TP + m) * H + k]; s.write(p); }
    };
    auto pull = [&](stream<vec<float, TP>>& s) {
        std::vector<float> a((size_t)S * H);
        for (int M = 0; M < S / TP; M++)
            for (int k = 0; k < H; k++) { auto p = s.read(); for (int m = 0; m < TP; m++) a[(size_t)(M * TP + m) * H + k] = p[m]; }
        return a;
    };
    bool ok = true;
    {   // RMSNorm
        stream<vec<float, TP>> in, out; stream<float> g;
        push(in, x); for (float v : gamma) g.write(v);
        pref_Layer_Norm<float, TP, HIDDEN_DIM>(in, g, out, S, H);
        auto y = pull(out);
        for (int t = 0; t < S; t++) {
            double ss = 0; for (int k = 0; k < H; k++) ss += (double)x[(size_t)t * H + k] * x[(size_t)t * H + k];
            const double rms = 1.0 / std::sqrt(ss / H + 1e-5);
            for (int k = 0; k < H; k++) if (std::abs(y[(size_t)t * H + k] - x[(size_t)t * H + k] * rms * gamma[k]) > 1e-5 * (1 + std::abs(y[(size_t)t * H + k]))) ok = false;
        }
    }
    {   // Swish, gate, residual
        stream<vec<float, TP>> in, sw, in2, gated, res_in, res_out;
        push(in, x); pref_Swish<float, TP, HIDDEN_DIM>(in, sw, S, H);
        push(in2, r); pref_Gate_Layer_fp32xfp32<TP, HIDDEN_DIM>(in2, sw, gated, S);
        push(res_in, x); pref_Residual_Layer<float, TP, HIDDEN_DIM>(gated, res_in, res_out, S);
        auto y = pull(res_out);
        for (size_t i = 0; i < y.size(); i++) {
            const double g = (double)x[i] / (1.0 + std::exp(-(double)x[i]));
            if (std::abs(y[i] - (r[i] * g + x[i])) > 1e-5 * (1 + std::abs(y[i]))) ok = false;
        }
    }
    {   // softmax rows
        stream<vec<float, TP>> in, out;
        push(in, x); pref_Softmax<float, TP, HIDDEN_DIM, 1024, 1>(in, out, S, H);
        auto y = pull(out);
        for (int t = 0; t < S; t++) {
            double mx = -1e300, sum = 0;
            for (int k = 0; k < H; k++) mx = std::max(mx, (double)x[(size_t)t * H + k]);
            for (int k = 0; k < H; k++) sum += std::exp(x[(size_t)t * H + k] - mx);
            for (int k = 0; k < H; k++) if (std::abs(y[(size_t)t * H + k] - std::exp(x[(size_t)t * H + k] - mx) / sum) > 1e-6) ok = false;
        }
    }
    verdict("RMSNorm / Swish / Gate / Residual / Softmax streams", ok);
}

static void pref_MHA_test() {
    const int S = 128, TP = TOKEN_PARALLEL;
    std::default_random_engine gen(42);
    std::uniform_real_distribution<float> dist(-128.0 / std::sqrt((double)HIDDEN_DIM), 128.0 / std::sqrt((double)HIDDEN_DIM));
    // the reference's documented synthetic scale fill (MHA_i8xi8.h:32-37, 467-472)
    std::vector<float> Q_s(Q_HEAD_NUM), K_s(KV_HEAD_NUM), V_s(KV_HEAD_NUM), A_s(Q_HEAD_NUM);
    for (int h = 0; h < Q_HEAD_NUM; h++) { Q_s[h] = float(h + 1) / HIDDEN_DIM; A_s[h] = 1.0f / 256; }
    for (int h = 0; h < KV_HEAD_NUM; h++) { K_s[h] = float(h + 1) / HIDDEN_DIM * 4; V_s[h] = float(h + 1) / HIDDEN_DIM * 4; }
    using VF = vec<float, TP>;
    std::vector<VF> q_mmap((size_t)S / TP * HIDDEN_DIM), k_mmap((size_t)S / TP * KV_HIDDEN_DIM), v_mmap((size_t)S / TP * KV_HIDDEN_DIM),
        o_mmap((size_t)S / TP * HIDDEN_DIM);
    std::vector<double> q_gold((size_t)S * HIDDEN_DIM), k_gold((size_t)S * KV_HIDDEN_DIM), v_gold((size_t)S * KV_HIDDEN_DIM);
    auto fq = [](double v, double scale, int lo, int hi) { int q = (int)std::round(v / scale); q = std::max(lo, std::min(hi, q)); return q * scale; };
    for (int i = 0; i < S; i++) {
        for (int h = 0; h < Q_HEAD_NUM; h++)
            for (int j = 0; j < HEAD_DIM; j++) {
                const float val = dist(gen);
                q_mmap[(size_t)(i / TP) * HIDDEN_DIM + h * HEAD_DIM + j][i % TP] = val;
                q_gold[(size_t)i * HIDDEN_DIM + h * HEAD_DIM + j] = fq((double)(val / (8.0f * Q_s[h])), 1.0, -128, 127) * Q_s[h];
            }
        for (int h = 0; h < KV_HEAD_NUM; h++)
            for (int j = 0; j < HEAD_DIM; j++) {
                const float kv = dist(gen), vv = dist(gen);
                k_mmap[(size_t)(i / TP) * KV_HIDDEN_DIM + h * HEAD_DIM + j][i % TP] = kv;
                v_mmap[(size_t)(i / TP) * KV_HIDDEN_DIM + h * HEAD_DIM + j][i % TP] = vv;
                k_gold[(size_t)i * KV_HIDDEN_DIM + h * HEAD_DIM + j] = fq((double)(kv / K_s[h]), 1.0, -128, 127) * K_s[h];
                v_gold[(size_t)i * KV_HIDDEN_DIM + h * HEAD_DIM + j] = fq((double)(vv / V_s[h]), 1.0, -128, 127) * V_s[h];
            }
    }
    std::cout << "kernel begins running!\n";
    const int64_t ns = MHA_i8xi8_Prefilling_layer<TP, Q_HEAD_NUM, KV_HEAD_NUM, HEAD_DIM>(q_mmap, k_mmap, v_mmap, o_mmap, Q_s.data(), K_s.data(),
                                                                                      V_s.data(), A_s.data(), S, 8.0f);
    std::cout << "kernel time: " << ns * 1e-9 << " s" << std::endl;
    bool correct = true;
    std::vector<double> a(S), p(S);
    for (int h = 0; h < Q_HEAD_NUM && correct; h++) {
        const int kh = h / (Q_HEAD_NUM / KV_HEAD_NUM);
        for (int i = 0; i < S && correct; i++) {
            double mx = -1e300, sum = 0;
            for (int j = 0; j <= i; j++) {
                double acc = 0;
                for (int d = 0; d < HEAD_DIM; d++) acc += q_gold[(size_t)i * HIDDEN_DIM + h * HEAD_DIM + d] * k_gold[(size_t)j * KV_HIDDEN_DIM + kh * HEAD_DIM + d];
                a[j] = acc; mx = std::max(mx, acc);
            }
            for (int j = 0; j <= i; j++) { p[j] = std::exp(a[j] - mx); sum += p[j]; }
            for (int j = 0; j <= i; j++) p[j] = std::min(255.0, std::round(p[j] / sum / A_s[h])) * A_s[h];
            for (int d = 0; d < HEAD_DIM; d++) {
                double o = 0;
                for (int j = 0; j <= i; j++) o += p[j] * v_gold[(size_t)j * KV_HIDDEN_DIM + kh * HEAD_DIM + d];
                const float my = o_mmap[(size_t)(i / TP) * HIDDEN_DIM + h * HEAD_DIM + d][i % TP];
                // the reference's criterion is 5e-3 relative; an absolute floor covers a probability byte that
                // rounds the other way between float and double arithmetic
                if (std::abs(my - o) > 5e-3 * std::abs(o) + 1.5 * A_s[h] * 128 * V_s[kh]) {
                    correct = false;
                    std::cout << "Mismatch at (" << i << ", " << h * HEAD_DIM + d << "): My: " << my << ", Ref: " << o << std::endl;
                    break;
                }
            }
        }
    }
    verdict("MHA (prefill, int8 q/k/v, uint8 probabilities)", correct);
}

int main() {
    try {
        QuantWrapper_Linear_Layer_q_decoding_test();
        QuantWrapper_Linear_Layer_q_decoding_w4a4_test();
        QuantWrapper_Linear_Layer_q_prefilling_test();
        FHT_test();
        Elementwise_test();
        pref_MHA_test();
    } catch (const std::exception& e) {
        std::cerr << "harness error: " << e.what() << std::endl;
        return 2;
    }
    return failures ? 1 : 0;
}

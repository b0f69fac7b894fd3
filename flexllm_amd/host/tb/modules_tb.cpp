// Testbench-style harness for the host-side module mirror (flexllm_modules.h), shaped like the reference's
// *_tb.cpp files: build seeded inputs in the stream packings, push them through the module functions, compare
// with an in-process golden, print a check mark or a cross.  Unlike the reference's harnesses the exit code is
// non-zero when a check fails.
//
//   QuantWrapper linear, decode   <-> SpinQuant_Llama_32_1B/Linear_Layer_Decoding_tb.cpp:93-251 (1e-2 relative)
//   QuantWrapper linear, prefill  <-> SpinQuant_Llama_32_1B/Linear_Layer_Prefilling_tb.cpp (1e-2 relative)
//   MHA prefill                   <-> SpinQuant_Llama_32_1B/MHA_i8xi8_prefilling_tb.cpp:12-268 (5e-3 relative)
//   MHA decode                    <-> SpinQuant_Llama_32_1B/MHA_i8xi8_decoding_tb.cpp:12-289 (QK^T 1e-3, attention 5e-3),
//                                     launched through fxhost::invoke(top, "hip", mmaps..., scalars...) on the reference's
//                                     own cache line layouts, and stage by stage through the dec_MHA_* module functions
//   layout adapters               <-> the packed int4 weight words and the KV-cache line layouts of the testbenches
//   QuantWrapper linear tops      <-> SpinQuant_Llama_32_1B/Linear_Layer_test.h:145-175, :332-364 launched through
//                                     fxhost::invoke on the testbenches' packed int4 weight words
//   Logits                        <-> Modules/Logits.h:34-279 (top-k layer, sampling + embedding feedback)
//   FHT / RMSNorm / Swish / residual / softmax / RoPE against float64 closed forms
#include <algorithm>
#include <array>
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

// Decode attention, shaped like SpinQuant_Llama_32_1B/MHA_i8xi8_decoding_tb.cpp:12-289 for one layer (layer 1 of 2, so
// that the layer offsets of the cache buffers matter): a history of PRE positions held in the reference's lane buffers,
// DEC tokens decoded on top.  Checks: (1) q.K^T of the last token against the fake-quant golden at 1e-3 through the
// dec_MHA_* module functions fed from the cache lines; (2) the whole attention through fxhost::invoke on the top
// function at 5e-3; (3) the module chain (scores -> softmax -> uint8 quant -> P.V -> dequant) against the top bit for bit.
static void dec_MHA_test() {
    constexpr int BP = 16, HP = 8, KP = 32, VP = 32, LAYERS = 2, LAYER = 1, MAX_SUM = 256, PRE = 100, DEC = 4;
    constexpr int H = HIDDEN_DIM, KV = KV_HIDDEN_DIM, per_q = H / BP, per_kv = KV / BP, hpl = KV_HEAD_NUM / HP;
    std::default_random_engine gen(42);
    std::uniform_real_distribution<float> dist(-128.0 / std::sqrt((double)HIDDEN_DIM), 128.0 / std::sqrt((double)HIDDEN_DIM));
    static float Q_s[LAYERS][Q_HEAD_NUM], K_s[LAYERS][KV_HEAD_NUM], V_s[LAYERS][KV_HEAD_NUM], A_s[LAYERS][Q_HEAD_NUM];
    for (int l = 0; l < LAYERS; l++) {
        for (int h = 0; h < Q_HEAD_NUM; h++) { Q_s[l][h] = float(h + 1 + l) / HIDDEN_DIM; A_s[l][h] = 1.0f / 256; }
        for (int h = 0; h < KV_HEAD_NUM; h++) { K_s[l][h] = float(h + 1 + l) / HIDDEN_DIM * 4; V_s[l][h] = float(h + 2 + l) / HIDDEN_DIM * 4; }
    }
    using VF = vec<float, BP>;
    using VK = vec<int8_t, KP>;
    using VV = vec<int8_t, VP>;
    std::vector<VF> q_mmap((size_t)DEC * per_q), k_mmap((size_t)(PRE + DEC) * per_kv), v_mmap((size_t)(PRE + DEC) * per_kv), o_mmap((size_t)DEC * per_q);
    std::vector<VK> k_caches[HP];
    std::vector<VV> v_caches[HP];
    for (int i = 0; i < HP; i++) {
        k_caches[i].assign((size_t)LAYERS * hpl * MAX_SUM / KP * HEAD_DIM, VK());
        v_caches[i].assign((size_t)LAYERS * hpl * HEAD_DIM / VP * MAX_SUM, VV());
    }
    std::vector<double> q_gold((size_t)DEC * H), k_gold((size_t)(PRE + DEC) * KV), v_gold((size_t)(PRE + DEC) * KV);
    for (int i = 0; i < DEC; i++)
        for (int j = 0; j < H; j++) {
            const float val = dist(gen);
            q_mmap[(size_t)i * per_q + j % per_q][j / per_q] = val;
            int qv = (int)std::round(val / 8.0f / Q_s[LAYER][j / HEAD_DIM]);
            qv = std::max(-128, std::min(127, qv));
            q_gold[(size_t)i * H + j] = qv * (double)Q_s[LAYER][j / HEAD_DIM];
        }
    for (int i = 0; i < PRE + DEC; i++)
        for (int j = 0; j < KV; j++) {
            const int h = j / HEAD_DIM, d = j % HEAD_DIM;
            const float kv = dist(gen), vv = dist(gen);
            k_mmap[(size_t)i * per_kv + j % per_kv][j / per_kv] = kv;
            v_mmap[(size_t)i * per_kv + j % per_kv][j / per_kv] = vv;
            int kq = std::max(-128, std::min(127, (int)std::round(kv / K_s[LAYER][h])));
            int vq = std::max(-128, std::min(127, (int)std::round(vv / V_s[LAYER][h])));
            if (i < PRE) {      // the history sits in the lane buffers, written with the testbench's own index formulas (:77-80, :214-216)
                k_caches[h / hpl][((size_t)(LAYER * hpl + h % hpl) * MAX_SUM + i) / KP * HEAD_DIM + d][i % KP] = (int8_t)kq;
                v_caches[h / hpl][((size_t)(LAYER * hpl + h % hpl) * HEAD_DIM + d) / VP * MAX_SUM + i][d % VP] = (int8_t)vq;
            }
            k_gold[(size_t)i * KV + j] = kq * (double)K_s[LAYER][h];
            v_gold[(size_t)i * KV + j] = vq * (double)V_s[LAYER][h];
        }
    std::cout << "kernel begins running!\n";
    const int64_t ns = invoke(MHA_i8xi8_decoding_layer<BP, HP, KP, VP, Q_HEAD_NUM, KV_HEAD_NUM, HEAD_DIM, VF, VK, VV>, "hip",
                              read_only_mmap(q_mmap), read_only_mmap(k_mmap), read_only_mmap(v_mmap), read_write_mmaps(k_caches),
                              read_write_mmaps(v_caches), write_only_mmap(o_mmap), Q_s[LAYER], K_s[LAYER], V_s[LAYER], A_s[LAYER], LAYER, LAYERS,
                              MAX_SUM, PRE, DEC, 8.0f);
    std::cout << "kernel time: " << ns * 1e-9 << " s" << std::endl;
    // (2) whole attention against the fake-quant golden
    bool correct = true;
    std::vector<double> a(PRE + DEC), p(PRE + DEC);
    for (int i = 0; i < DEC && correct; i++)
        for (int h = 0; h < Q_HEAD_NUM && correct; h++) {
            const int kh = h / (Q_HEAD_NUM / KV_HEAD_NUM), len = PRE + i + 1;
            double mx = -1e300, sum = 0;
            for (int j = 0; j < len; j++) {
                double acc = 0;
                for (int d = 0; d < HEAD_DIM; d++) acc += q_gold[(size_t)i * H + h * HEAD_DIM + d] * k_gold[(size_t)j * KV + kh * HEAD_DIM + d];
                a[j] = acc; mx = std::max(mx, acc);
            }
            for (int j = 0; j < len; j++) { p[j] = std::exp(a[j] - mx); sum += p[j]; }
            for (int j = 0; j < len; j++) p[j] = std::min(255.0, std::round(p[j] / sum / A_s[LAYER][h])) * A_s[LAYER][h];
            for (int d = 0; d < HEAD_DIM; d++) {
                double o = 0;
                for (int j = 0; j < len; j++) o += p[j] * v_gold[(size_t)j * KV + kh * HEAD_DIM + d];
                const int jj = h * HEAD_DIM + d;
                const float my = o_mmap[(size_t)i * per_q + jj % per_q][jj / per_q];
                if (std::abs(my - o) > 5e-3 * std::abs(o) + 1.5 * A_s[LAYER][h] * 128 * V_s[LAYER][kh]) {
                    correct = false;
                    std::cout << "Mismatch at (" << i << ", " << jj << "): My: " << my << ", Ref: " << o << std::endl;
                    break;
                }
            }
        }
    verdict("MHA (decode, the reference's cache lines, launched through invoke)", correct);
    // the decoded rows were written back into the lane buffers: layer 0's block untouched, layer 1 holds PRE + DEC rows
    {
        bool ok = true;
        std::vector<int8_t> k_tm((size_t)(PRE + DEC) * KV), v_tm((size_t)(PRE + DEC) * KV);
        const CacheGeom geom{LAYERS, KV_HEAD_NUM, HEAD_DIM, MAX_SUM};
        kcache_decode_to_token_major<HP, KP>(k_caches, geom, LAYER, PRE + DEC, k_tm.data());
        vcache_decode_to_token_major<HP, VP>(v_caches, geom, LAYER, PRE + DEC, v_tm.data());
        for (int i = 0; i < PRE + DEC; i++)
            for (int j = 0; j < KV; j++) {
                if (std::abs(k_tm[(size_t)i * KV + j] * (double)K_s[LAYER][j / HEAD_DIM] - k_gold[(size_t)i * KV + j]) > 1e-9) ok = false;
                if (std::abs(v_tm[(size_t)i * KV + j] * (double)V_s[LAYER][j / HEAD_DIM] - v_gold[(size_t)i * KV + j]) > 1e-9) ok = false;
            }
        std::vector<int8_t> k0((size_t)MAX_SUM * KV);
        kcache_decode_to_token_major<HP, KP>(k_caches, geom, 0, MAX_SUM, k0.data());
        for (int8_t v : k0) if (v != 0) ok = false;
        verdict("decode cache write-back (rows of the decoded tokens in the reference's line layout)", ok);
    }
    // (1) + (3): the last decoded token stage by stage through the module functions, keys and values streamed from the lane buffers
    {
        const int t = DEC - 1, len = PRE + DEC, per = Q_HEAD_NUM / HP, padded = (len + KP - 1) / KP * KP;
        stream<vec<float, HP>> q_s;
        stream<vec<int8_t, HP>> q8_s;
        std::vector<float> qv(H);
        for (int j = 0; j < H; j++) qv[j] = q_mmap[(size_t)t * per_q + j % per_q][j / per_q];
        for (int Hh = 0; Hh < per; Hh++)
            for (int k = 0; k < HEAD_DIM; k++) { vec<float, HP> pk; for (int m = 0; m < HP; m++) pk[m] = qv[(size_t)(m * per + Hh) * HEAD_DIM + k]; q_s.write(pk); }
        dec_MHA_static_sym_per_tensor_quant_layer_fp32_qint<8, HP, HEAD_DIM, Q_HEAD_NUM, true, LAYERS>(q_s, q8_s, Q_s, LAYER, HEAD_DIM, 8.0f);
        // key streams in the cache manager's read order (Modules/MHA.h:503-513): per lane, its heads, each repeated for the
        // group's query heads; lane i of the q.K^T module serves query heads i*per + Hh, i.e. KV head (i*per + Hh) / 4
        std::array<stream<VK>, HP> k_str;
        for (int Hh = 0; Hh < per; Hh++)
            for (int N = 0; N < padded / KP; N++)
                for (int k = 0; k < HEAD_DIM; k++)
                    for (int i = 0; i < HP; i++) {
                        const int kh = (i * per + Hh) / (Q_HEAD_NUM / KV_HEAD_NUM);
                        k_str[i].write(k_caches[kh / hpl][((size_t)(LAYER * hpl + kh % hpl) * MAX_SUM + N * KP) / KP * HEAD_DIM + k]);
                    }
        stream<vec<int32_t, HP>> acc_s, acc_trim;
        dec_MHA_i8xi8_qxk_template<HP, KP, Q_HEAD_NUM, HEAD_DIM, 6, MAX_SUM>(q8_s, k_str, acc_s, len);
        for (int Hh = 0; Hh < per; Hh++)                                   // dec_quant_a_discard_template: drop the padded keys
            for (int k = 0; k < padded; k++) { auto pk = acc_s.read(); if (k < len) acc_trim.write(pk); }
        stream<vec<float, HP>> a_s, sfm_s;
        dec_MHA_static_sym_per_tensor_dequant_layer_qint_fp32<22, HP, MAX_SUM, Q_HEAD_NUM, KV_HEAD_NUM, LAYERS>(acc_trim, a_s, Q_s, K_s, LAYER, len);
        // (1) scores against the golden at 1e-3 (MHA_i8xi8_decoding_tb.cpp: qxk check)
        bool ok1 = true;
        std::vector<float> scores((size_t)Q_HEAD_NUM * len);
        stream<vec<float, HP>> a_copy;
        for (int Hh = 0; Hh < per; Hh++)
            for (int k = 0; k < len; k++) { auto pk = a_s.read(); a_copy.write(pk); for (int m = 0; m < HP; m++) scores[(size_t)(m * per + Hh) * len + k] = pk[m]; }
        for (int h = 0; h < Q_HEAD_NUM; h++)
            for (int j = 0; j < len; j++) {
                double g = 0;
                const int kh = h / (Q_HEAD_NUM / KV_HEAD_NUM);
                for (int d = 0; d < HEAD_DIM; d++) g += q_gold[(size_t)t * H + h * HEAD_DIM + d] * k_gold[(size_t)j * KV + kh * HEAD_DIM + d];
                if (std::abs(scores[(size_t)h * len + j] - g) > 1e-3 * std::abs(g) + 1e-6) ok1 = false;
            }
        verdict("MHA q.K^T (decode modules fed from the cache lines, 1e-3)", ok1);
        dec_MHA_Softmax<float, HP, MAX_SUM, Q_HEAD_NUM>(a_copy, sfm_s, len);
        stream<vec<uint8_t, HP>> p8_s;
        dec_MHA_static_sym_per_tensor_quant_layer_fp32_qint<8, HP, MAX_SUM, Q_HEAD_NUM, false, LAYERS>(sfm_s, p8_s, A_s, LAYER, len, 1.0f);
        std::array<stream<VV>, HP> v_str;
        for (int Hh = 0; Hh < per; Hh++)
            for (int N = 0; N < HEAD_DIM / VP; N++)
                for (int k = 0; k < len; k++)
                    for (int i = 0; i < HP; i++) {
                        const int kh = (i * per + Hh) / (Q_HEAD_NUM / KV_HEAD_NUM);
                        v_str[i].write(v_caches[kh / hpl][((size_t)(LAYER * hpl + kh % hpl) * HEAD_DIM + N * VP) / VP * MAX_SUM + k]);
                    }
        stream<vec<int32_t, HP>> o_acc_s;
        stream<vec<float, HP>> o_s;
        dec_MHA_i8xi8_axv_template<HP, VP, Q_HEAD_NUM, HEAD_DIM, MAX_SUM, 8, true>(p8_s, v_str, o_acc_s, len);
        dec_MHA_static_sym_per_tensor_dequant_layer_qint_fp32<24, HP, HEAD_DIM, Q_HEAD_NUM, KV_HEAD_NUM, LAYERS>(o_acc_s, o_s, A_s, V_s, LAYER, HEAD_DIM);
        bool ok3 = true;
        int differing = 0;
        for (int Hh = 0; Hh < per; Hh++)
            for (int k = 0; k < HEAD_DIM; k++) {
                auto pk = o_s.read();
                for (int m = 0; m < HP; m++) {
                    const int h = m * per + Hh, jj = h * HEAD_DIM + k;
                    const float d = std::abs(pk[m] - o_mmap[(size_t)t * per_q + jj % per_q][jj / per_q]);
                    // identical integer stages; the two softmax sums are associated differently, so a probability byte on a
                    // rounding tie may differ by one step (a whole head's 64 outputs then move by at most A_s * 128 * V_s)
                    if (d != 0) differing++;
                    if (d > 1.5f * A_s[LAYER][h] * 128 * V_s[LAYER][h / (Q_HEAD_NUM / KV_HEAD_NUM)]) ok3 = false;
                }
            }
        if (differing > 2 * HEAD_DIM) ok3 = false;
        verdict("MHA module chain (scores, softmax, uint8 probabilities, P.V, dequant) against the fused top", ok3);
    }
}

// Prefill attention stage by stage through the module functions against the fused top, and the decode RoPE module.
static void pref_MHA_modules_test() {
    constexpr int S = 32, TP = TOKEN_PARALLEL, QH = 4, KVH = 2, KP = 16, VP = 16, LAYERS = 1;
    constexpr int Hd = QH * HEAD_DIM, KVd = KVH * HEAD_DIM;
    std::default_random_engine gen(5);
    std::uniform_real_distribution<float> dist(-2.8f, 2.8f);
    static float Q_s[LAYERS][QH], K_s[LAYERS][KVH], V_s[LAYERS][KVH], A_s[LAYERS][QH];
    for (int h = 0; h < QH; h++) { Q_s[0][h] = 0.004f + 0.001f * h; A_s[0][h] = 1.0f / 255; }
    for (int h = 0; h < KVH; h++) { K_s[0][h] = 0.03f + 0.002f * h; V_s[0][h] = 0.025f + 0.003f * h; }
    using VF = vec<float, TP>;
    std::vector<VF> q_mmap((size_t)S / TP * Hd), k_mmap((size_t)S / TP * KVd), v_mmap((size_t)S / TP * KVd), o_mmap((size_t)S / TP * Hd);
    for (auto& pk : q_mmap) for (int m = 0; m < TP; m++) pk[m] = dist(gen);
    for (auto& pk : k_mmap) for (int m = 0; m < TP; m++) pk[m] = dist(gen);
    for (auto& pk : v_mmap) for (int m = 0; m < TP; m++) pk[m] = dist(gen);
    MHA_i8xi8_Prefilling_layer<TP, QH, KVH, HEAD_DIM>(q_mmap, k_mmap, v_mmap, o_mmap, Q_s[0], K_s[0], V_s[0], A_s[0], S, 8.0f);
    // stage chain: static quant -> q.K^T -> dequant -> mask -> softmax -> uint8 quant -> P.V -> dequant
    stream<VF> q_in, k_in, v_in;
    for (auto& pk : q_mmap) q_in.write(pk);
    for (auto& pk : k_mmap) k_in.write(pk);
    for (auto& pk : v_mmap) v_in.write(pk);
    stream<vec<int8_t, TP>> q8_s, k8_s, v8_s;
    pref_static_sym_per_tensor_quant_layer_fp32_qint<8, TP, HEAD_DIM, QH, true, 1024, LAYERS>(q_in, q8_s, Q_s, 0, S, HEAD_DIM, 8.0f);
    pref_static_sym_per_tensor_quant_layer_fp32_qint<8, TP, HEAD_DIM, KVH, true, 1024, LAYERS>(k_in, k8_s, K_s, 0, S, HEAD_DIM, 1.0f);
    pref_static_sym_per_tensor_quant_layer_fp32_qint<8, TP, HEAD_DIM, KVH, true, 1024, LAYERS>(v_in, v8_s, V_s, 0, S, HEAD_DIM, 1.0f);
    std::vector<int8_t> k8((size_t)S * KVd), v8((size_t)S * KVd);
    for (int M = 0; M < S / TP; M++)
        for (int j = 0; j < KVd; j++) {
            auto kp = k8_s.read(); auto vp = v8_s.read();
            for (int m = 0; m < TP; m++) { k8[(size_t)(M * TP + m) * KVd + j] = kp[m]; v8[(size_t)(M * TP + m) * KVd + j] = vp[m]; }
        }
    // key / value streams in the prefill cache managers' read order (Modules/MHA.h:96-106, :322-333)
    stream<vec<int8_t, KP>> k_str;
    stream<vec<int8_t, VP>> v_str;
    for (int M = 0; M < S / TP; M++)
        for (int h = 0; h < QH; h++) {
            const int kh = h / (QH / KVH);
            for (int N = 0; N < S / KP; N++)
                for (int d = 0; d < HEAD_DIM; d++) { vec<int8_t, KP> pk; for (int j = 0; j < KP; j++) pk[j] = k8[(size_t)(N * KP + j) * KVd + kh * HEAD_DIM + d]; k_str.write(pk); }
            for (int N = 0; N < HEAD_DIM / VP; N++)
                for (int t = 0; t < S; t++) { vec<int8_t, VP> pk; for (int j = 0; j < VP; j++) pk[j] = v8[(size_t)t * KVd + kh * HEAD_DIM + N * VP + j]; v_str.write(pk); }
        }
    stream<vec<int32_t, TP>> acc_s, o_acc_s;
    stream<VF> a_s, masked_s, sfm_s, o_s;
    stream<vec<uint8_t, TP>> p8_s;
    pref_MHA_i8xi8_qxk_template<TP, KP, QH, HEAD_DIM, 6, 1024>(q8_s, k_str, acc_s, S);
    pref_static_sym_per_tensor_dequant_layer_qint_fp32<22, TP, 1024, QH, KVH, 1024, LAYERS>(acc_s, a_s, Q_s, K_s, 0, S, S);
    pref_causal_mask_template<float, TP, 1024, 1024, QH>(a_s, masked_s, S, S);
    pref_Softmax<float, TP, 1024, 1024, QH>(masked_s, sfm_s, S, S);
    pref_static_sym_per_tensor_quant_layer_fp32_qint<8, TP, 1024, QH, false, 1024, LAYERS>(sfm_s, p8_s, A_s, 0, S, S, 1.0f);
    pref_MHA_i8xi8_axv_template<TP, VP, QH, HEAD_DIM, 1024, 10, true>(p8_s, v_str, o_acc_s, S);
    pref_static_sym_per_tensor_dequant_layer_qint_fp32<26, TP, HEAD_DIM, QH, KVH, 1024, LAYERS>(o_acc_s, o_s, A_s, V_s, 0, S, HEAD_DIM);
    bool ok = true;
    int flips = 0;
    for (size_t i = 0; i < o_mmap.size(); i++) {
        auto pk = o_s.read();
        for (int m = 0; m < TP; m++) {
            const float d = std::abs(pk[m] - o_mmap[i][m]);
            if (d != 0) flips++;                                            // the row sums of the two paths are associated differently:
            if (d > 1.5f * A_s[0][0] * 128 * 0.04f) ok = false;             // a probability byte on a tie may differ by one step
        }
    }
    if (flips > (int)(o_mmap.size() * TP) / 20) ok = false;
    verdict("MHA module chain (prefill: q.K^T, mask, softmax, uint8 probabilities, P.V) against the fused top", ok);
    // decode RoPE module against the closed form
    {
        constexpr int HP = 8, POS = 37;
        static float PE_sin[64][HEAD_DIM / 2], PE_cos[64][HEAD_DIM / 2];
        for (int s0 = 0; s0 < 64; s0++)
            for (int i = 0; i < HEAD_DIM / 2; i++) { const double f = std::pow(500000.0, -2.0 * i / HEAD_DIM); PE_sin[s0][i] = (float)std::sin(s0 * f); PE_cos[s0][i] = (float)std::cos(s0 * f); }
        std::vector<float> x((size_t)Q_HEAD_NUM * HEAD_DIM);
        for (auto& v : x) v = dist(gen);
        stream<vec<float, HP>> in, out;
        const int per = Q_HEAD_NUM / HP;
        for (int Hh = 0; Hh < per; Hh++)
            for (int k = 0; k < HEAD_DIM; k++) { vec<float, HP> pk; for (int m = 0; m < HP; m++) pk[m] = x[(size_t)(m * per + Hh) * HEAD_DIM + k]; in.write(pk); }
        dec_RoPE_layer<float, HP, HEAD_DIM, Q_HEAD_NUM, 64>(in, out, PE_sin, PE_cos, Q_HEAD_NUM, POS);
        bool okr = true;
        for (int Hh = 0; Hh < per; Hh++)
            for (int k = 0; k < HEAD_DIM; k++) {
                auto pk = out.read();
                for (int m = 0; m < HP; m++) {
                    const float* xh = &x[(size_t)(m * per + Hh) * HEAD_DIM];
                    const int kk = k % 32;
                    const double e = k < 32 ? (double)xh[kk] * PE_cos[POS][kk] - (double)xh[kk + 32] * PE_sin[POS][kk]
                                            : (double)xh[kk] * PE_sin[POS][kk] + (double)xh[kk + 32] * PE_cos[POS][kk];
                    if (std::abs(pk[m] - e) > 1e-5) okr = false;
                }
            }
        verdict("RoPE (decode stream, head-parallel lanes)", okr);
    }
}

// The layout adapters against the testbenches' index formulas, and as round trips.
static void adapters_test() {
    bool ok = true;
    std::default_random_engine gen(9);
    std::uniform_int_distribution<int> d4(-8, 7), d8(-128, 127);
    {   // int4 weight words, decode form (Linear_Layer_Decoding_tb.cpp:176-186) and prefill form (Linear_Layer.h:134-185)
        constexpr int N = 256, K = 64, BP = 8, WP = 16;
        std::vector<int8_t> w((size_t)N * K), back((size_t)N * K);
        for (auto& v : w) v = (int8_t)d4(gen);
        std::vector<vec<int8_t, WP / 2>> lanes[BP];
        pack_weight_int4_decode<WP, BP>(w.data(), N, K, lanes);
        for (int n : {0, 1, 17, 31, 32, 255})
            for (int k : {0, 5, 63}) {
                const int I = n / (N / BP), i = n % (N / BP);
                const unsigned byte = (uint8_t)lanes[I][(size_t)(i / WP) * K + k][(i / 2) % (WP / 2)];
                if (sext4(byte >> (4 * (i % 2))) != w[(size_t)n * K + k]) ok = false;
            }
        unpack_weight_int4_decode<WP, BP>(lanes, N, K, back.data());
        if (back != w) ok = false;
        std::vector<vec<int8_t, WP / 2>> flat;
        pack_weight_int4_prefill<WP>(w.data(), N, K, flat);
        for (int n : {0, 3, 16, 200})
            for (int k : {0, 63}) {
                const unsigned byte = (uint8_t)flat[(size_t)(n / WP) * K + k][(n / 2) % (WP / 2)];
                if (sext4(byte >> (4 * (n % 2))) != w[(size_t)n * K + k]) ok = false;
            }
        std::fill(back.begin(), back.end(), 0);
        unpack_weight_int4_prefill<WP>(flat, N, K, back.data());
        if (back != w) ok = false;
    }
    {   // KV cache lines, prefill buffers (Modules/MHA.h:74-109, :299-336)
        constexpr int L = 2, KVH = 2, HD = 64, SMAX = 64, KP = 16, VP = 16, LEN = 40, LAYER = 1;
        const CacheGeom g{L, KVH, HD, SMAX};
        std::vector<int8_t> tm((size_t)LEN * KVH * HD), back(tm.size());
        for (auto& v : tm) v = (int8_t)d8(gen);
        std::vector<vec<int8_t, KP>> kc((size_t)L * KVH * SMAX / KP * HD);
        std::vector<vec<int8_t, VP>> vcv((size_t)L * KVH * HD / VP * SMAX);
        kcache_prefill_from_token_major<KP>(tm.data(), g, LAYER, 0, LEN, kc);
        vcache_prefill_from_token_major<VP>(tm.data(), g, LAYER, 0, LEN, vcv);
        for (int t : {0, 15, 16, 39})
            for (int h = 0; h < KVH; h++)
                for (int d : {0, 17, 63}) {
                    if (kc[((size_t)(LAYER * KVH + h) * SMAX / KP + t / KP) * HD + d][t % KP] != tm[((size_t)t * KVH + h) * HD + d]) ok = false;
                    const int ch = h * HD + d;
                    if (vcv[((size_t)LAYER * (KVH * HD) / VP + ch / VP) * SMAX + t][ch % VP] != tm[((size_t)t * KVH + h) * HD + d]) ok = false;
                }
        kcache_prefill_to_token_major<KP>(kc, g, LAYER, LEN, back.data());
        if (back != tm) ok = false;
        vcache_prefill_to_token_major<VP>(vcv, g, LAYER, LEN, back.data());
        if (back != tm) ok = false;
    }
    verdict("layout adapters (packed int4 weight words, prefill KV-cache lines; the decode lines are exercised by the MHA test)", ok);
}


// The linear testbench tops launched the way the testbenches launch them - fxhost::invoke(top, "hip", mmaps..., length) -
// on the testbenches' own buffers: activations in the stream packings and the packed int4 weight words written with
// the index formulas of Linear_Layer_Decoding_tb.cpp:176-186 and Linear_Layer_Prefilling_tb.cpp:226-231 (not through
// this build's pack adapters).  Checked against the quantised golden of the testbench (q_out * s_x * s_w + b_x * sum_w,
// :236-249) to fp32 rounding and against its fake-quant golden at its own 1e-2.
template <bool DECODE>
static void QuantWrapper_Linear_Layer_q_tops_test() {
    constexpr int K = HIDDEN_DIM, N = HIDDEN_DIM, BP = T_BLOCK_PARALLEL, TP = TOKEN_PARALLEL;
    constexpr int WP = DECODE ? DEC_W_PARALLEL : 24, WPR = DECODE ? DEC_W_PARALLEL : 32;   // prefill: PRE_QKVO_W_PARALLEL = 24, read width 32
    const int T = DECODE ? 8 : 64;
    std::default_random_engine gen(42);
    std::uniform_real_distribution<float> dist(-1.0, 1.0);
    using VF = vec<float, DECODE ? BP : TP>;
    using VW = vec<int8_t, WPR / 2>;
    using VS = vec<float, 2>;
    std::vector<float> x((size_t)T * K), fq((size_t)T * K), in_s(T), in_b(T), w_fq((size_t)N * K);
    std::vector<int> q_in((size_t)T * K), q_w((size_t)N * K);
    std::vector<VF> input_mmap(DECODE ? (size_t)T * K / BP : (size_t)T / TP * K), output_mmap(DECODE ? (size_t)T * N / BP : (size_t)T / TP * N);
    for (int i = 0; i < T; i++) {
        float vmax = -1e30f, vmin = 1e30f;
        for (int j = 0; j < K; j++) {
            const float val = dist(gen);
            x[(size_t)i * K + j] = val; vmax = std::max(vmax, val); vmin = std::min(vmin, val);
            if (DECODE) input_mmap[(size_t)i * (K / BP) + j % (K / BP)][j / (K / BP)] = val;
            else input_mmap[(size_t)(i / TP) * K + j][i % TP] = val;
        }
        float scale = (vmax - vmin) / 15.0f;
        if (scale == 0) scale = 1.0f;
        in_s[i] = scale; in_b[i] = vmin;
        for (int j = 0; j < K; j++) {
            const int q = (int)std::round((x[(size_t)i * K + j] - vmin) / scale);
            q_in[(size_t)i * K + j] = q;
            fq[(size_t)i * K + j] = q * scale + vmin;
        }
    }
    std::vector<VS> weight_s_sum_mmap(N);
    std::vector<VW> lanes[BP], flat;
    if (DECODE) for (int I = 0; I < BP; I++) lanes[I].assign((size_t)(N / BP + WP - 1) / WP * K, VW());
    else flat.assign((size_t)((N + WP - 1) / WP) * K, VW());
    for (int n = 0; n < N; n++) {
        float w_max = 0;
        for (int j = 0; j < K; j++) { w_fq[(size_t)n * K + j] = dist(gen); w_max = std::max(w_max, std::abs(w_fq[(size_t)n * K + j])); }
        float scale = w_max / 7.0f;
        if (scale == 0) scale = 1.0f;
        weight_s_sum_mmap[n][0] = scale; weight_s_sum_mmap[n][1] = 0;
        for (int j = 0; j < K; j++) {
            int qval = (int)std::round(w_fq[(size_t)n * K + j] / scale);
            qval = std::max(-8, std::min(7, qval));
            w_fq[(size_t)n * K + j] = qval * scale;
            q_w[(size_t)n * K + j] = qval;
            weight_s_sum_mmap[n][1] += w_fq[(size_t)n * K + j];
            // the packed word this value lives in, by the testbench's formula
            int8_t* slot;
            int nib;
            if (DECODE) { const int I = n / (N / BP), i = n % (N / BP); slot = &lanes[I][(size_t)(i / WP) * K + j][(i / 2) % (WP / 2)]; nib = i % 2; }
            else { slot = &flat[(size_t)((n / 2) / (WP / 2)) * K + j][(n / 2) % (WP / 2)]; nib = n % 2; }
            const unsigned old = (uint8_t)*slot, v = (unsigned)qval & 0xF;
            *slot = (int8_t)(nib ? ((old & 0x0F) | (v << 4)) : ((old & 0xF0) | v));
        }
    }
    std::cout << "kernel begins running!\n";
    int64_t ns;
    if constexpr (DECODE)
        ns = invoke(QuantWrapper_Linear_Layer_q_Decoding_layer<BP, WP, K, N, VF, VW, VS>, "hip", read_only_mmap(input_mmap),
                    read_only_mmaps(lanes), read_only_mmap(weight_s_sum_mmap), write_only_mmap(output_mmap), T);
    else
        ns = invoke(QuantWrapper_Linear_Layer_q_Prefilling_layer<TP, WP, K, N, VF, VW, VS>, "hip", read_only_mmap(input_mmap),
                    read_only_mmap(flat), read_only_mmap(weight_s_sum_mmap), write_only_mmap(output_mmap), T);
    std::cout << "kernel time: " << ns * 1e-9 << " s" << std::endl;
    bool correct = true;
    double worst_q = 0;
    for (int i = 0; i < T && correct; i++)
        for (int j = 0; j < N; j++) {
            long long acc = 0;
            double gold_fq = 0;
            for (int k = 0; k < K; k++) {
                acc += (long long)q_in[(size_t)i * K + k] * q_w[(size_t)j * K + k];
                gold_fq += (double)fq[(size_t)i * K + k] * w_fq[(size_t)j * K + k];
            }
            const float gold_q = (float)acc * in_s[i] * weight_s_sum_mmap[j][0] + in_b[i] * weight_s_sum_mmap[j][1];
            const float my = DECODE ? output_mmap[(size_t)i * (N / BP) + j % (N / BP)][j / (N / BP)] : output_mmap[(size_t)(i / TP) * N + j][i % TP];
            worst_q = std::max(worst_q, (double)std::abs(my - gold_q));
            if (std::abs(my - gold_q) > 1e-5 * std::abs(gold_q) + 1e-5 || std::abs(my - gold_fq) > 1e-2 * std::abs(gold_fq) + 1e-3) {
                correct = false;
                std::cout << "Mismatch at (" << i << ", " << j << "): My: " << my << ", Ref_q: " << gold_q << ", Ref_fq: " << gold_fq << std::endl;
                break;
            }
        }
    verdict(DECODE ? "QuantWrapper linear top (decode) through invoke on the testbench's packed int4 weight lanes"
                   : "QuantWrapper linear top (prefill, weight parallel 24 in words of 32) through invoke on the testbench's packed int4 weight words", correct);
}

// pref_Linear_Layer_i4xi4 as a module: uint4 activations in the prefill packing x resident int4 weights -> exact int32
static void pref_Linear_Layer_i4xi4_test() {
    constexpr int S = 32, K = 256, N = 96, TP = TOKEN_PARALLEL;
    std::default_random_engine gen(5);
    std::uniform_int_distribution<int> da(0, 15), dw(-8, 7);
    std::vector<int> a((size_t)S * K), w((size_t)N * K);
    std::vector<int8_t> w8((size_t)N * K);
    for (auto& v : a) v = da(gen);
    for (size_t i = 0; i < w.size(); i++) { w[i] = dw(gen); w8[i] = (int8_t)w[i]; }
    stream<vec<uint8_t, TP>> in;
    stream<vec<int32_t, TP>> out;
    for (int M = 0; M < S / TP; M++)
        for (int k = 0; k < K; k++) { vec<uint8_t, TP> p; for (int m = 0; m < TP; m++) p[m] = (uint8_t)a[(size_t)(M * TP + m) * K + k]; in.write(p); }
    DeviceWeight4 weight(w8.data(), N, K);
    pref_Linear_Layer_i4xi4<TP, 24, K, 8, N, S, true>(in, weight, out, S, K, N);
    bool ok = true;
    for (int M = 0; M < S / TP; M++)
        for (int n = 0; n < N; n++) {
            const auto p = out.read();
            for (int m = 0; m < TP; m++) {
                int acc = 0;
                for (int k = 0; k < K; k++) acc += a[(size_t)(M * TP + m) * K + k] * w[(size_t)n * K + k];
                if (p[m] != acc) ok = false;
            }
        }
    verdict("pref_Linear_Layer_i4xi4 (uint4 x int4, prefill stream packing, exact int32)", ok && out.empty());
}

// Modules/Logits.h: top-k layer and the sampling + embedding layer on block-partitioned logit streams
static void Logits_test() {
    constexpr int BPS = 8, V = 128256, TOPK = 5;
    std::default_random_engine gen(11);
    std::normal_distribution<float> nd(0.0f, 2.0f);
    std::vector<float> logits(V);
    for (auto& v : logits) v = nd(gen);
    logits[777] = logits[90001];                                   // an exact tie somewhere in the body of the distribution
    std::vector<int> order(V);
    for (int i = 0; i < V; i++) order[i] = i;
    std::partial_sort(order.begin(), order.begin() + TOPK, order.end(), [&](int a, int b) { return logits[a] > logits[b] || (logits[a] == logits[b] && a < b); });
    double e[TOPK], sum = 0;
    for (int k = 0; k < TOPK; k++) { e[k] = std::exp((double)logits[order[k]] - (double)logits[order[0]]); sum += e[k]; }
    auto feed = [&](stream<vec<float, BPS>>& s, const std::vector<float>& l, int n) {
        for (int m = 0; m < n / BPS; m++) { vec<float, BPS> p; for (int i = 0; i < BPS; i++) p[i] = l[(size_t)i * (n / BPS) + m]; s.write(p); }
    };
    bool ok = true;
    {
        stream<vec<float, BPS>> ls;
        stream<vec<float, 2>> out;
        feed(ls, logits, V);
        dec_Logits_Max_K_Layer<float, BPS, V, TOPK>(ls, out, V);
        for (int k = 0; k < TOPK; k++) {
            const auto p = out.read();
            if ((int)p[0] != order[k] || std::abs(p[1] - e[k] / sum) > 1e-5) { ok = false; std::cout << "top-k " << k << ": My: " << p[0] << " " << p[1] << ", Ref: " << order[k] << " " << e[k] / sum << std::endl; }
        }
        ok = ok && out.empty();
    }
    {   // sampling + embedding feedback on a small vocabulary (the table is a host buffer here), several uniform numbers
        constexpr int V2 = 4096, HID = 256, BPE = 8;
        std::vector<float> l2(logits.begin(), logits.begin() + V2);
        std::vector<int> o2(V2);
        for (int i = 0; i < V2; i++) o2[i] = i;
        std::partial_sort(o2.begin(), o2.begin() + TOPK, o2.end(), [&](int a, int b) { return l2[a] > l2[b] || (l2[a] == l2[b] && a < b); });
        float pr[TOPK], part[2] = {0, 0};
        for (int k = 0; k < TOPK; k++) { pr[k] = std::exp(l2[o2[k]] - l2[o2[0]]); part[k % 2] += pr[k]; }   // Logits.h:231-246, float like the reference
        const float tot = part[0] + part[1];
        float cdf[TOPK];
        for (int k = 0; k < TOPK; k++) { pr[k] /= tot; cdf[k] = k ? pr[k] + cdf[k - 1] : pr[0]; }
        std::vector<vec<float, BPE>> vocab_lib((size_t)V2 * HID / BPE);
        for (size_t i = 0; i < vocab_lib.size(); i++) for (int j = 0; j < BPE; j++) vocab_lib[i][j] = (float)(i * BPE + j) * 0.25f;
        for (float r : {0.0f, 0.37f, 0.62f, 0.81f, 0.93f, 0.9999f}) {
            bool near_edge = false;
            for (int k = 0; k < TOPK; k++) near_edge = near_edge || std::abs(cdf[k] - r) < 1e-5f;
            if (near_edge) continue;                                 // the device's expf against glibc's at a boundary
            int sel = TOPK - 1;
            for (int k = TOPK - 1; k >= 0; k--) if (r < cdf[k]) sel = k;
            stream<vec<float, BPS>> ls;
            stream<vec<float, BPE>> emb;
            feed(ls, l2, V2);
            int sampled_idx = -1;
            dec_Sampling_Embedding_Layer<float, BPS, V2, TOPK, BPE, HID>(ls, vocab_lib, emb, r, sampled_idx, V2, HID);
            if (sampled_idx != o2[sel]) { ok = false; std::cout << "rand " << r << ": My: " << sampled_idx << ", Ref: " << o2[sel] << std::endl; }
            for (int i = 0; i < HID / BPE && sampled_idx >= 0; i++) {
                const auto p = emb.read();
                for (int j = 0; j < BPE; j++) if (p[j] != vocab_lib[(size_t)sampled_idx * (HID / BPE) + i][j]) ok = false;
            }
            ok = ok && emb.empty();
        }
    }
    verdict("Logits (top-k layer on 128256 logits; sampling + embedding feedback)", ok);
}

int main() {
    try {
        QuantWrapper_Linear_Layer_q_decoding_test();
        QuantWrapper_Linear_Layer_q_decoding_w4a4_test();
        QuantWrapper_Linear_Layer_q_prefilling_test();
        FHT_test();
        Elementwise_test();
        pref_MHA_test();
        dec_MHA_test();
        pref_MHA_modules_test();
        adapters_test();
        QuantWrapper_Linear_Layer_q_tops_test<true>();
        QuantWrapper_Linear_Layer_q_tops_test<false>();
        pref_Linear_Layer_i4xi4_test();
        Logits_test();
    } catch (const std::exception& e) {
        std::cerr << "harness error: " << e.what() << std::endl;
        return 2;
    }
    return failures ? 1 : 0;
}

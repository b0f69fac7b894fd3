// Test helper (host only): reads a `parameters/` directory the way the reference's testbench does and dumps what it
// saw as raw binary, so that a Python test can compare it with the arrays the directory was written from.
//
// What is mirrored, from SpinQuant_Llama_32_1B/SpinQuant_Prefilling_Decoding_mem_opt_tb.cpp:
//   * the generated headers are #include'd INSIDE a function body (:435-443) and indexed as
//     w_<proj>_s[layer][out], w_<proj>_sum[layer][out] (:445-478), w_lm_head_lm_head_s[v], w_lm_head_lm_head_sum[v]
//     (:716-719), RMSNorm_weight[2*layer (+1)][hidden] and RMSNorm_weight[2*layers][hidden] (:480-486, :724-736);
//   * Q_s.h / K_s.h / V_s.h / A_s.h are #include'd at file scope (SpinQuant_Llama_32_1B/MHA_i8xi8.h:11-14) and passed
//     as `const float input_s[layers][heads]` (Modules/quant.h:252-261);
//   * weight files are opened as "parameters/<proj>_L%02d.bin" and read one output row at a time with
//     seekg(row * input_dim) + read(input_dim bytes) (:30-47, :187-217), the embedding file as fp32 rows with
//     seekg(token * hidden * 4) (:150-172), lm_head.bin without a layer suffix (:196-201).
// The dimensions come in as -D macros (FX_LAYERS, FX_HIDDEN, FX_KV_HIDDEN, FX_INTER, FX_Q_HEADS, FX_KV_HEADS, FX_VOCAB);
// the program runs with the directory that holds `parameters/` as its working directory.
#include <cstdint>
#include <cstdio>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "parameters/Q_s.h"
#include "parameters/K_s.h"
#include "parameters/V_s.h"
#include "parameters/A_s.h"

static FILE* out_file;

static void dump(const void* p, size_t bytes) { fwrite(p, 1, bytes, out_file); }

// a consumer shaped like pref_static_sym_per_tensor_quant_layer_fp32_qint's scale argument
template <int L, int HEADS>
static void dump_static(const float input_s[L][HEADS]) {
    for (int l = 0; l < L; l++)
        for (int h = 0; h < HEADS; h++) dump(&input_s[l][h], sizeof(float));
}

static bool dump_weight_rows(const std::string& layer_name, int layer, int input_dim, int output_dim) {
    char name[256];
    if (layer_name == "lm_head") std::snprintf(name, sizeof(name), "parameters/%s.bin", layer_name.c_str());
    else std::snprintf(name, sizeof(name), "parameters/%s_L%02d.bin", layer_name.c_str(), layer);
    std::ifstream fin(name, std::ios::binary);
    if (!fin) { std::cerr << "Failed to open file: " << name << "\n"; return false; }
    // two output channels per iteration, each read with its own seek, as the testbench's packers do
    for (int n = 0; n < output_dim / 2; ++n) {
        std::vector<int8_t> data_0(input_dim), data_1(input_dim);
        fin.seekg(static_cast<std::streamoff>(2 * n) * input_dim, std::ios::beg);
        fin.read(reinterpret_cast<char*>(data_0.data()), data_0.size());
        if (!fin) { std::cerr << "Read error @ row " << 2 * n << " in " << name << "\n"; return false; }
        fin.seekg(static_cast<std::streamoff>(2 * n + 1) * input_dim, std::ios::beg);
        fin.read(reinterpret_cast<char*>(data_1.data()), data_1.size());
        if (!fin) { std::cerr << "Read error @ row " << 2 * n + 1 << " in " << name << "\n"; return false; }
        dump(data_0.data(), data_0.size());
        dump(data_1.data(), data_1.size());
    }
    return true;
}

static bool dump_embedding_rows(const std::vector<int>& token_idx, int hidden_dim) {
    std::ifstream fin("parameters/model_embed_tokens_fp32.bin", std::ios::binary);
    if (!fin) { std::cerr << "Failed to open the embedding file\n"; return false; }
    for (int tok : token_idx) {
        std::vector<float> data(hidden_dim);
        fin.seekg(static_cast<std::streamoff>(tok) * hidden_dim * sizeof(float), std::ios::beg);
        fin.read(reinterpret_cast<char*>(data.data()), data.size() * sizeof(float));
        if (!fin) { std::cerr << "Read error @ token_idx " << tok << "\n"; return false; }
        dump(data.data(), data.size() * sizeof(float));
    }
    return true;
}

int main(int argc, char** argv) {
    if (argc < 2) return 2;
    out_file = fopen(argv[1], "wb");
    if (!out_file) return 2;
    const bool with_head = argc > 2 && std::string(argv[2]) == "head";

    #include "parameters/w_k_proj_s_sum.h"
    #include "parameters/w_v_proj_s_sum.h"
    #include "parameters/w_q_proj_s_sum.h"
    #include "parameters/w_o_proj_s_sum.h"
    #include "parameters/w_gate_proj_s_sum.h"
    #include "parameters/w_up_proj_s_sum.h"
    #include "parameters/w_down_proj_s_sum.h"
#ifdef FX_WITH_HEAD
    #include "parameters/w_lm_head_lm_head.h"
#endif
    #include "parameters/w_rmsnorm.h"

    // section 1: scale / sum pairs in the order q, k, v, o, gate, up, down; per layer, per output channel: {s, sum}
#define FX_DUMP_PAIRS(S, SUM, N)                                   \
    for (int i = 0; i < FX_LAYERS; i++)                            \
        for (int j = 0; j < (N); j++) {                            \
            const float pair[2] = {S[i][j], SUM[i][j]};            \
            dump(pair, sizeof(pair));                              \
        }
    FX_DUMP_PAIRS(w_q_proj_s, w_q_proj_sum, FX_HIDDEN)
    FX_DUMP_PAIRS(w_k_proj_s, w_k_proj_sum, FX_KV_HIDDEN)
    FX_DUMP_PAIRS(w_v_proj_s, w_v_proj_sum, FX_KV_HIDDEN)
    FX_DUMP_PAIRS(w_o_proj_s, w_o_proj_sum, FX_HIDDEN)
    FX_DUMP_PAIRS(w_gate_proj_s, w_gate_proj_sum, FX_INTER)
    FX_DUMP_PAIRS(w_up_proj_s, w_up_proj_sum, FX_INTER)
    FX_DUMP_PAIRS(w_down_proj_s, w_down_proj_sum, FX_HIDDEN)
    // section 2: the norm weights, rows 2i and 2i+1 per layer, then the final row
    for (int i = 0; i < FX_LAYERS; i++)
        for (int j = 0; j < FX_HIDDEN; j++) {
            const float two[2] = {RMSNorm_weight[2 * i][j], RMSNorm_weight[2 * i + 1][j]};
            dump(two, sizeof(two));
        }
    for (int j = 0; j < FX_HIDDEN; j++) dump(&RMSNorm_weight[2 * FX_LAYERS][j], sizeof(float));
    // section 3: static attention scales
    dump_static<FX_LAYERS, FX_Q_HEADS>(Q_s);
    dump_static<FX_LAYERS, FX_KV_HEADS>(K_s);
    dump_static<FX_LAYERS, FX_KV_HEADS>(V_s);
    dump_static<FX_LAYERS, FX_Q_HEADS>(A_s);
    // section 4: weight rows of every projection and layer
    const struct { const char* name; int in, out; } proj[7] = {
        {"q_proj", FX_HIDDEN, FX_HIDDEN}, {"k_proj", FX_HIDDEN, FX_KV_HIDDEN}, {"v_proj", FX_HIDDEN, FX_KV_HIDDEN},
        {"o_proj", FX_HIDDEN, FX_HIDDEN}, {"gate_proj", FX_HIDDEN, FX_INTER}, {"up_proj", FX_HIDDEN, FX_INTER},
        {"down_proj", FX_INTER, FX_HIDDEN}};
    for (const auto& p : proj)
        for (int l = 0; l < FX_LAYERS; l++)
            if (!dump_weight_rows(p.name, l, p.in, p.out)) return 1;
    // section 5: embedding rows of a few token ids, fetched by seeking like the testbench's embedding reader
    if (!dump_embedding_rows({FX_VOCAB - 1, 0, 5, FX_VOCAB / 2}, FX_HIDDEN)) return 1;
    // section 6 (4-bit exports): the output head's rows and its scale / sum pairs
#ifdef FX_WITH_HEAD
    if (with_head) {
        if (!dump_weight_rows("lm_head", 0, FX_HIDDEN, FX_VOCAB)) return 1;
        for (int j = 0; j < FX_VOCAB; j++) {
            const float pair[2] = {w_lm_head_lm_head_s[j], w_lm_head_lm_head_sum[j]};
            dump(pair, sizeof(pair));
        }
    }
#endif
    (void)with_head;
    fclose(out_file);
    return 0;
}

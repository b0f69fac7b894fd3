// Layout adapters between the reference's host buffers (the "mmap" vectors its testbenches fill) and the dense
// token-major / row-major arrays of the C ABI.  Pure permutations, written from the index formulas of the reference's
// own testbenches and loaders; every function has an inverse so that a harness can round-trip.
//
//   weights   packed int4, two output channels per byte, WP channels per word, K-major inside a channel block:
//               prefill  W_mmap[(n/WP)*K + k][(n/2) % (WP/2)], nibble n%2          (Modules/Linear_Layer.h:134-185)
//               decode   W_mmaps[I][(i/WP)*K + k][(i/2) % (WP/2)], nibble i%2, n = I*N/BP + i
//                                                        (SpinQuant_Llama_32_1B/Linear_Layer_Decoding_tb.cpp:176-186)
//             <-> int8 [N][K] row-major, one value per byte (the on-disk parameters/<proj>_L%02d.bin form and the ABI's)
//   KV cache  prefill  K  k_cache[((l*KVH + h)*Smax/KP + t/KP)*64 + d][t%KP]       (Modules/MHA.h:74-109)
//                      V  v_cache[(l*KVH*64/VP + ch/VP)*Smax + t][ch%VP], ch = h*64+d (Modules/MHA.h:299-336)
//             decode   K  k_caches[h/(KVH/HP)][((l*KVH/HP + h%(KVH/HP))*Smax + t)/KP*64 + d][t%KP]
//                      V  v_caches[h/(KVH/HP)][((l*KVH/HP + h%(KVH/HP))*64 + d)/VP*Smax + t][d%VP]
//                                                        (SpinQuant_Llama_32_1B/MHA_i8xi8_decoding_tb.cpp:77-80, :214-216)
//             <-> int8 [t][kv_head][64] token-major, the input of flexllm_kv_store_i8
#pragma once
#include <cstddef>
#include <cstdint>
#include <vector>

namespace fxhost {

inline int8_t sext4(unsigned v) { return (int8_t)((v & 8) ? (int)(v & 0xF) - 16 : (int)(v & 0xF)); }

// ---- int4 weight words ------------------------------------------------------------------------------------------
// VEC: a vector of WP/2 bytes (hls::vector<ap_int<8>, WP/2> or fxhost::vec<int8_t, WP/2>), indexable with [].
template <int WP, class VEC>
void unpack_weight_int4_prefill(const std::vector<VEC>& w_mmap, int n_dim, int k_dim, int8_t* row_major) {
    for (int n = 0; n < n_dim; n++)
        for (int k = 0; k < k_dim; k++) {
            const unsigned byte = (unsigned)(uint8_t)(int)w_mmap[(size_t)(n / WP) * k_dim + k][(n / 2) % (WP / 2)];
            row_major[(size_t)n * k_dim + k] = sext4(byte >> (4 * (n % 2)));
        }
}
template <int WP, class VEC>
void pack_weight_int4_prefill(const int8_t* row_major, int n_dim, int k_dim, std::vector<VEC>& w_mmap) {
    w_mmap.assign((size_t)((n_dim + WP - 1) / WP) * k_dim, VEC());
    for (int n = 0; n < n_dim; n++)
        for (int k = 0; k < k_dim; k++) {
            auto& slot = w_mmap[(size_t)(n / WP) * k_dim + k][(n / 2) % (WP / 2)];
            const unsigned old = (unsigned)(uint8_t)(int)slot, v = (unsigned)row_major[(size_t)n * k_dim + k] & 0xF;
            slot = (int8_t)(n % 2 ? ((old & 0x0F) | (v << 4)) : ((old & 0xF0) | v));
        }
}
// decode: BP lane buffers, lane I holds output channels I*N/BP .. (I+1)*N/BP - 1
template <int WP, int BP, class VEC>
void unpack_weight_int4_decode(const std::vector<VEC>* w_mmaps, int n_dim, int k_dim, int8_t* row_major) {
    const int per = n_dim / BP;
    for (int I = 0; I < BP; I++)
        for (int i = 0; i < per; i++)
            for (int k = 0; k < k_dim; k++) {
                const unsigned byte = (unsigned)(uint8_t)(int)w_mmaps[I][(size_t)(i / WP) * k_dim + k][(i / 2) % (WP / 2)];
                row_major[(size_t)(I * per + i) * k_dim + k] = sext4(byte >> (4 * (i % 2)));
            }
}
template <int WP, int BP, class VEC>
void pack_weight_int4_decode(const int8_t* row_major, int n_dim, int k_dim, std::vector<VEC>* w_mmaps) {
    const int per = n_dim / BP;
    for (int I = 0; I < BP; I++) {
        w_mmaps[I].assign((size_t)((per + WP - 1) / WP) * k_dim, VEC());
        for (int i = 0; i < per; i++)
            for (int k = 0; k < k_dim; k++) {
                auto& slot = w_mmaps[I][(size_t)(i / WP) * k_dim + k][(i / 2) % (WP / 2)];
                const unsigned old = (unsigned)(uint8_t)(int)slot, v = (unsigned)row_major[(size_t)(I * per + i) * k_dim + k] & 0xF;
                slot = (int8_t)(i % 2 ? ((old & 0x0F) | (v << 4)) : ((old & 0xF0) | v));
            }
    }
}

// ---- KV cache lines ---------------------------------------------------------------------------------------------
struct CacheGeom {
    int layers, kv_heads, head_dim, max_seq;     // max_seq = MAX_PRE_SEQ_LEN (prefill buffers) or MAX_SUM_SEQ_LEN (decode buffers)
};

// prefill buffers -> token-major int8 [len][kv_heads][head_dim] of one layer, and one token range back
template <int KP, class VEC>
void kcache_prefill_to_token_major(const std::vector<VEC>& k_cache, const CacheGeom& g, int layer, int len, int8_t* out) {
    for (int t = 0; t < len; t++)
        for (int h = 0; h < g.kv_heads; h++)
            for (int d = 0; d < g.head_dim; d++)
                out[((size_t)t * g.kv_heads + h) * g.head_dim + d] =
                    (int8_t)(int)k_cache[((size_t)(layer * g.kv_heads + h) * (g.max_seq / KP) + t / KP) * g.head_dim + d][t % KP];
}
template <int KP, class VEC>
void kcache_prefill_from_token_major(const int8_t* in, const CacheGeom& g, int layer, int t0, int len, std::vector<VEC>& k_cache) {
    for (int t = t0; t < t0 + len; t++)
        for (int h = 0; h < g.kv_heads; h++)
            for (int d = 0; d < g.head_dim; d++)
                k_cache[((size_t)(layer * g.kv_heads + h) * (g.max_seq / KP) + t / KP) * g.head_dim + d][t % KP] =
                    in[((size_t)(t - t0) * g.kv_heads + h) * g.head_dim + d];
}
template <int VP, class VEC>
void vcache_prefill_to_token_major(const std::vector<VEC>& v_cache, const CacheGeom& g, int layer, int len, int8_t* out) {
    const int kvd = g.kv_heads * g.head_dim;
    for (int t = 0; t < len; t++)
        for (int ch = 0; ch < kvd; ch++)
            out[(size_t)t * kvd + ch] = (int8_t)(int)v_cache[((size_t)layer * (kvd / VP) + ch / VP) * g.max_seq + t][ch % VP];
}
template <int VP, class VEC>
void vcache_prefill_from_token_major(const int8_t* in, const CacheGeom& g, int layer, int t0, int len, std::vector<VEC>& v_cache) {
    const int kvd = g.kv_heads * g.head_dim;
    for (int t = t0; t < t0 + len; t++)
        for (int ch = 0; ch < kvd; ch++)
            v_cache[((size_t)layer * (kvd / VP) + ch / VP) * g.max_seq + t][ch % VP] = in[(size_t)(t - t0) * kvd + ch];
}

// decode buffers: HP lane buffers, lane h / (kv_heads/HP) holds KV head h
template <int HP, int KP, class VEC>
void kcache_decode_to_token_major(const std::vector<VEC>* k_caches, const CacheGeom& g, int layer, int len, int8_t* out) {
    const int hpl = g.kv_heads / HP;                  // heads per lane buffer
    for (int t = 0; t < len; t++)
        for (int h = 0; h < g.kv_heads; h++)
            for (int d = 0; d < g.head_dim; d++)
                out[((size_t)t * g.kv_heads + h) * g.head_dim + d] =
                    (int8_t)(int)k_caches[h / hpl][((size_t)(layer * hpl + h % hpl) * g.max_seq + t) / KP * g.head_dim + d][t % KP];
}
template <int HP, int KP, class VEC>
void kcache_decode_from_token_major(const int8_t* in, const CacheGeom& g, int layer, int t0, int len, std::vector<VEC>* k_caches) {
    const int hpl = g.kv_heads / HP;
    for (int t = t0; t < t0 + len; t++)
        for (int h = 0; h < g.kv_heads; h++)
            for (int d = 0; d < g.head_dim; d++)
                k_caches[h / hpl][((size_t)(layer * hpl + h % hpl) * g.max_seq + t) / KP * g.head_dim + d][t % KP] =
                    in[((size_t)(t - t0) * g.kv_heads + h) * g.head_dim + d];
}
template <int HP, int VP, class VEC>
void vcache_decode_to_token_major(const std::vector<VEC>* v_caches, const CacheGeom& g, int layer, int len, int8_t* out) {
    const int hpl = g.kv_heads / HP;
    for (int t = 0; t < len; t++)
        for (int h = 0; h < g.kv_heads; h++)
            for (int d = 0; d < g.head_dim; d++)
                out[((size_t)t * g.kv_heads + h) * g.head_dim + d] =
                    (int8_t)(int)v_caches[h / hpl][((size_t)(layer * hpl + h % hpl) * g.head_dim + d) / VP * g.max_seq + t][d % VP];
}
template <int HP, int VP, class VEC>
void vcache_decode_from_token_major(const int8_t* in, const CacheGeom& g, int layer, int t0, int len, std::vector<VEC>* v_caches) {
    const int hpl = g.kv_heads / HP;
    for (int t = t0; t < t0 + len; t++)
        for (int h = 0; h < g.kv_heads; h++)
            for (int d = 0; d < g.head_dim; d++)
                v_caches[h / hpl][((size_t)(layer * hpl + h % hpl) * g.head_dim + d) / VP * g.max_seq + t][d % VP] =
                    in[((size_t)(t - t0) * g.kv_heads + h) * g.head_dim + d];
}

}  // namespace fxhost

// C ABI entry points; the kernels live in attn_decode_kernels.h.
#include "attn_decode_kernels.h"

using namespace fx;

extern "C" {

int flexllm_kv_append_i8(const float* k, const float* v, int8_t* k_cache, int8_t* v_cache, const flexllm_mha_scales* sc,
                         int tokens, int kv_heads, int head_dim, int max_pos, int pos0, void* stream) {
    FX_REQUIRE(k && v && k_cache && v_cache && sc && sc->k_s && sc->v_s, "kv_append: null pointer");
    FX_REQUIRE(head_dim == kHd, "kv_append: head_dim=%d (only 64)", head_dim);
    FX_REQUIRE(tokens >= 0 && kv_heads > 0 && max_pos % kVBlock == 0 && pos0 >= 0 && pos0 + tokens <= max_pos,
               "kv_append: tokens=%d pos0=%d max_pos=%d (max_pos %% 64 == 0, pos0+tokens <= max_pos)", tokens, pos0, max_pos);
    if (tokens == 0) return FLEXLLM_OK;
    const size_t n = (size_t)tokens * kv_heads * kHd;
    const int grid = (int)((n + 255) / 256 > 2048 ? 2048 : (n + 255) / 256);
    kv_append_kernel<<<grid, 256, 0, as_stream(stream)>>>(k, v, k_cache, v_cache, sc->k_s, sc->v_s, tokens, kv_heads, max_pos, pos0);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_kv_store_i8(const int8_t* k8, const int8_t* v8, int8_t* k_cache, int8_t* v_cache, int tokens, int kv_heads,
                        int head_dim, int max_pos, int pos0, void* stream) {
    FX_REQUIRE(k8 && v8 && k_cache && v_cache, "kv_store: null pointer");
    FX_REQUIRE(head_dim == kHd, "kv_store: head_dim=%d (only 64)", head_dim);
    FX_REQUIRE(tokens >= 0 && kv_heads > 0 && max_pos % kVBlock == 0 && pos0 >= 0 && pos0 + tokens <= max_pos,
               "kv_store: tokens=%d pos0=%d max_pos=%d (max_pos %% 64 == 0, pos0+tokens <= max_pos)", tokens, pos0, max_pos);
    if (tokens == 0) return FLEXLLM_OK;
    const size_t n = (size_t)tokens * kv_heads * kHd;
    const int grid = (int)((n + 255) / 256 > 2048 ? 2048 : (n + 255) / 256);
    kv_store_kernel<<<grid, 256, 0, as_stream(stream)>>>(k8, v8, k_cache, v_cache, tokens, kv_heads, max_pos, pos0);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_mha_i8_decode(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache, const flexllm_mha_scales* sc,
                          float* o, uint8_t* p8_out, int len, int q_heads, int kv_heads, int head_dim, int max_pos,
                          void* stream) {
    FX_REQUIRE(q8 && k_cache && v_cache && sc && o, "mha_decode: null pointer");
    FX_REQUIRE(sc->q_s && sc->k_s && sc->v_s && sc->a_s, "mha_decode: null scale table");
    FX_REQUIRE(head_dim == kHd, "mha_decode: head_dim=%d (only 64)", head_dim);
    FX_REQUIRE(kv_heads > 0 && q_heads % kv_heads == 0 && q_heads / kv_heads >= 1 && q_heads / kv_heads <= 4,
               "mha_decode: q_heads=%d kv_heads=%d (group size 1..4)", q_heads, kv_heads);
    FX_REQUIRE(len >= 1 && len <= kChunk * kMaxChunks && len <= max_pos && max_pos % kVBlock == 0,
               "mha_decode: len=%d max_pos=%d (1 <= len <= 8192, len <= max_pos, max_pos %% 64 == 0)", len, max_pos);
    int rc = ensure_scratch(q_heads, len);
    if (rc) return rc;
    return mha_decode_launch(q8, k_cache, v_cache, sc->q_s, sc->k_s, sc->v_s, sc->a_s, o, p8_out, g_scratch.scores,
                             g_scratch.stats, g_scratch.o_acc, len, q_heads, kv_heads, max_pos, as_stream(stream));
}

}  // extern "C"

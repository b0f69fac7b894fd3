// C ABI entry points; the kernels live in attn_decode_kernels.h.
#include "attn_decode_kernels.h"

using namespace fx;

namespace {

// Scratch of the entry point that allocates nothing: scores [32 heads][8192 keys] fp32, chunk statistics [32][64]
// float2, attention accumulators [32][64] int32, in device memory that belongs to the loaded library (one copy per
// GPU, held until the process ends).  In host code `na_scratch` only names the symbol; the address a kernel can use
// is looked up once per device and kept in na_ptr.
constexpr int kNaHeads = 32;
constexpr int kNaLen = kChunk * kMaxChunks;
constexpr size_t kNaScoreBytes = (size_t)kNaHeads * kNaLen * sizeof(float);
constexpr size_t kNaStatBytes = (size_t)kNaHeads * kMaxChunks * sizeof(float2);
constexpr size_t kNaAccBytes = (size_t)kNaHeads * kHd * sizeof(int32_t);
static __device__ __align__(256) unsigned char na_scratch[kNaScoreBytes + kNaStatBytes + kNaAccBytes];
constexpr int kNaMaxDevices = 64;
unsigned char* na_ptr[kNaMaxDevices] = {};
std::mutex na_mu;

int na_scratch_of_current_device(unsigned char** out) {
    int dev = 0;
    FX_HIP(hipGetDevice(&dev));
    FX_REQUIRE(dev >= 0 && dev < kNaMaxDevices, "mha_decode_noalloc: device index %d (at most %d devices)", dev, kNaMaxDevices);
    std::lock_guard<std::mutex> lk(na_mu);
    if (!na_ptr[dev]) {
        void* p = nullptr;
        FX_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(na_scratch)));
        FX_REQUIRE(p != nullptr, "mha_decode_noalloc: the scratch symbol has no address on device %d", dev);
        na_ptr[dev] = static_cast<unsigned char*>(p);
    }
    *out = na_ptr[dev];
    return FLEXLLM_OK;
}

}  // namespace

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
    DecodeScratch ds;
    int rc = decode_scratch_of_stream(as_stream(stream), q_heads, len, &ds);
    if (rc) return rc;
    return mha_decode_launch(q8, k_cache, v_cache, sc->q_s, sc->k_s, sc->v_s, sc->a_s, o, p8_out, ds.scores, ds.stats,
                             ds.o_acc, len, q_heads, kv_heads, max_pos, as_stream(stream));
}

int flexllm_mha_i8_decode_noalloc(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache, const flexllm_mha_scales* sc,
                                  float* o, uint8_t* p8_out, int len, int q_heads, int kv_heads, int head_dim, int max_pos,
                                  void* stream) {
    FX_REQUIRE(q8 && k_cache && v_cache && sc && o, "mha_decode_noalloc: null pointer");
    FX_REQUIRE(sc->q_s && sc->k_s && sc->v_s && sc->a_s, "mha_decode_noalloc: null scale table");
    FX_REQUIRE(head_dim == kHd, "mha_decode_noalloc: head_dim=%d (only 64)", head_dim);
    FX_REQUIRE(kv_heads > 0 && q_heads % kv_heads == 0 && q_heads / kv_heads >= 1 && q_heads / kv_heads <= 4,
               "mha_decode_noalloc: q_heads=%d kv_heads=%d (group size 1..4)", q_heads, kv_heads);
    FX_REQUIRE(q_heads <= kNaHeads, "mha_decode_noalloc: q_heads=%d exceeds the built-in scratch (at most %d heads)", q_heads, kNaHeads);
    FX_REQUIRE(len >= 1 && len <= kNaLen, "mha_decode_noalloc: len=%d exceeds the built-in scratch (1..%d keys)", len, kNaLen);
    FX_REQUIRE(len <= max_pos && max_pos % kVBlock == 0, "mha_decode_noalloc: len=%d max_pos=%d (len <= max_pos, max_pos %% 64 == 0)",
               len, max_pos);
    unsigned char* base = nullptr;
    int rc = na_scratch_of_current_device(&base);
    if (rc) return rc;
    // Nothing here has to start at zero: the score kernel clears the accumulators of the heads it serves, and scores and
    // chunk statistics are written for every key below len before they are read.
    return mha_decode_launch(q8, k_cache, v_cache, sc->q_s, sc->k_s, sc->v_s, sc->a_s, o, p8_out, reinterpret_cast<float*>(base),
                             reinterpret_cast<float2*>(base + kNaScoreBytes),
                             reinterpret_cast<int32_t*>(base + kNaScoreBytes + kNaStatBytes), len, q_heads, kv_heads, max_pos,
                             as_stream(stream));
}

}  // extern "C"

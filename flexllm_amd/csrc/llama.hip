// Llama-3.2-1B W8A8 SpinQuant graph on one GPU: owns the repacked weights, the int8 KV cache and the
// activation workspace, and strings the kernels together in the reference's layer order
// (RMSNorm -> quant -> q/k/v -> RoPE -> static int8 quant -> KV append -> int8 attention -> o_proj -> residual
//  -> RMSNorm -> quant -> gate/up -> SiLU*up -> Hadamard R4 -> quant -> down -> residual).
//
// Decode keeps every per-step quantity that changes between steps (position, current token) in device
// memory so that one captured HIP graph can be replayed for every generated token.
#include "attn_decode_kernels.h"
#include "elementwise_kernels.h"
#include "fht_kernels.h"
#include "gemv_i8.h"
#include "logits_kernels.h"
#include "decode_mega.h"
#include "die_arena.h"
#include "prefill.h"
#include <atomic>
#include <vector>

struct flexllm_llama {
    flexllm_llama_config cfg;
    std::vector<fx::LayerW> layers;
    float* gamma = nullptr;
    float *q_s = nullptr, *k_s = nullptr, *v_s = nullptr, *a_s = nullptr;
    float *rope_sin = nullptr, *rope_cos = nullptr;
    uint16_t* embed = nullptr;
    int8_t *k_cache = nullptr, *v_cache = nullptr;   // [layers] x per-layer cache
    size_t cache_layer_bytes = 0;
    // decode workspace
    float *x = nullptr, *x2 = nullptr, *qkv = nullptr, *h = nullptr, *nrm = nullptr, *logits = nullptr;
    int8_t *xq = nullptr, *q8 = nullptr;
    float* xs = nullptr;
    float* scores = nullptr;
    float2* stats = nullptr;
    // Persistent kernel: the words its workgroups hand to each other, one copy per I/O die, in 8 KiB blocks of `arena`
    // ([die][block]; see die_arena.h).  Tagged arrays start as 0xFF..FF (never a live tag), accumulators and barrier as 0.
    fx::DieArena arena;
    unsigned long long xblk[2][2] = {};        // MegaParams::xblk: which arena block holds block k of die d's copy
    void* xptr[2][fx::kXbCount] = {};          // the same as pointers (host-side resets)
    int32_t* o_acc = nullptr;
    int* state = nullptr;           // [0] position of the token being processed, [1] step index
    float* am_v = nullptr;
    int* am_i = nullptr;
    float* topk_val = nullptr;      // sampler: per-workgroup candidates of the first selection stage
    int* topk_idx = nullptr;
    float* gen_x = nullptr;         // generate: embeddings of the prompt, [gen_rows][hidden] (allocated on first use)
    int gen_rows = 0;
    int* gen_token = nullptr;       // generate: the token fed back between decode steps
    hipGraphExec_t graph_exec = nullptr;
    int* graph_token_io = nullptr;
    int* graph_tokens_out = nullptr;
    hipStream_t graph_stream = nullptr;
    std::vector<void*> owned;
    fx::PrefillWorkspace pws;
    fx::LayerW* layers_dev = nullptr;   // device copy of `layers` for the persistent kernel
    // W4A4 model (flexllm_llama_create_w4a4): the nibble-packed matrices with their row sums, the int4 output head
    bool w4 = false;
    std::vector<fx::LayerW4> layers4;
    fx::LayerW4* layers4_dev = nullptr;
    uint8_t* head_w4 = nullptr;
    float *head_s = nullptr, *head_sum = nullptr;
    bool mega_ok = false;               // shapes match the persistent kernel's compile-time constants
    int decode_mode = 0;                // 0: persistent kernel when possible, 1: one kernel per stage
    long long* timeline = nullptr;      // stage stamps of the persistent kernel (debug aid)
};

namespace fx {

// ---- small fused decode kernels ------------------------------------------------------------------
// Dequantise the attention accumulators and quantise the 2048-vector per token for o_proj; one block.
template <int VPT>
static __global__ __launch_bounds__(256) void dec_out_quant_kernel(const int32_t* __restrict__ o_acc, const float* __restrict__ a_s,
                                                                   const float* __restrict__ v_s, int8_t* __restrict__ q,
                                                                   float* __restrict__ s, int n, int group) {
    __shared__ float red[4];
    float v[VPT];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * 256;
        v[i] = 0.0f;
        if (idx < n) {
            const int qh = idx / kHd;
            v[i] = (float)o_acc[idx] * a_s[qh] * v_s[qh / group];
            amax = fmaxf(amax, fabsf(v[i]));
        }
    }
    amax = block_max<4>(amax, red);
    const float sc = sym_scale_127_uniform(amax);
    if (threadIdx.x == 0) s[0] = sc;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * 256;
        if (idx < n) q[idx] = (int8_t)quant_round(v[i], sc);
    }
}

static __global__ void set_state_kernel(int* state, int pos, int step) { state[0] = pos; state[1] = step; }

static __global__ __launch_bounds__(64) void argmax_final_advance_kernel(const float* __restrict__ pv, const int* __restrict__ pi,
                                                                         int nparts, int* __restrict__ token_io,
                                                                         int* __restrict__ tokens_out, int* __restrict__ state) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < nparts; i += 64) {
        const float v = pv[i];
        const int idx = pi[i];
        if (v > best || (v == best && idx < bi)) { best = v; bi = idx; }
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        const float ov = __shfl_xor(best, m);
        const int oi = __shfl_xor(bi, m);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (threadIdx.x == 0) {
        const int tok = bi == 0x7fffffff ? 0 : bi;
        token_io[0] = tok;
        tokens_out[state[1]] = tok;
        state[0] += 1;
        state[1] += 1;
    }
}

static int dev_alloc(flexllm_llama* m, void** p, size_t bytes) {
    hipError_t e = hipMalloc(p, bytes ? bytes : 1);
    if (e != hipSuccess) {
        set_error("hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        return e == hipErrorOutOfMemory ? FLEXLLM_ENOMEM : FLEXLLM_EHIP;
    }
    m->owned.push_back(*p);
    return FLEXLLM_OK;
}
#define FX_ALLOC(m, ptr, bytes)                                    \
    do {                                                           \
        int rc_ = dev_alloc(m, (void**)&(ptr), (bytes));           \
        if (rc_) return rc_;                                       \
    } while (0)

// All decode kernels of one layer, enqueued on `st`.
static int decode_layer(flexllm_llama* m, int l, hipStream_t st) {
    const flexllm_llama_config& c = m->cfg;
    const LayerW& w = m->layers[l];
    const int H = c.hidden, KV = c.kv_hidden, I = c.inter;
    const int group = c.q_heads / c.kv_heads;
    const float* g0 = m->gamma + (size_t)(2 * l) * H;
    const float* g1 = m->gamma + (size_t)(2 * l + 1) * H;
    const float* q_s = m->q_s + (size_t)l * c.q_heads;
    const float* k_s = m->k_s + (size_t)l * c.kv_heads;
    const float* v_s = m->v_s + (size_t)l * c.kv_heads;
    const float* a_s = m->a_s + (size_t)l * c.q_heads;
    int8_t* kc = m->k_cache + (size_t)l * m->cache_layer_bytes;
    int8_t* vc = m->v_cache + (size_t)l * m->cache_layer_bytes;
    int rc;
    // attention block
    rmsnorm_kernel<1, true, 512><<<1, 512, 0, st>>>(m->x, g0, nullptr, m->xq, m->xs, H, c.eps);
    if ((rc = launch_gemv<kEpiDequant>(m->xq, w.wqkv, nullptr, m->xs, w.sqkv, nullptr, m->qkv, H, H + 2 * KV, st))) return rc;
    qkv_post_kernel<<<1, 256, 0, st>>>(m->qkv, m->rope_sin, m->rope_cos, q_s, k_s, v_s, m->q8, kc, vc, m->state, 0,
                                       c.q_heads, c.kv_heads, c.max_pos);
    dim3 grid(c.max_pos / kChunk, c.kv_heads);
    dec_scores_kernel<<<grid, 64 * group, 0, st>>>(m->q8, kc, q_s, k_s, m->scores, m->stats, m->o_acc, m->state, 0,
                                                   c.max_pos, group, c.max_pos);
    dec_pv_kernel<<<grid, 64 * group, 0, st>>>(m->scores, m->stats, vc, a_s, m->o_acc, nullptr, m->state, 0, c.max_pos,
                                               group, c.max_pos);
    dec_out_quant_kernel<8><<<1, 256, 0, st>>>(m->o_acc, a_s, v_s, m->xq, m->xs, H, group);
    if ((rc = launch_gemv<kEpiDequant>(m->xq, w.wo, nullptr, m->xs, w.so, m->x, m->x2, H, H, st))) return rc;
    // feed-forward block
    rmsnorm_kernel<1, true, 512><<<1, 512, 0, st>>>(m->x2, g1, nullptr, m->xq, m->xs, H, c.eps);
    if ((rc = launch_gemv<kEpiSwiglu>(m->xq, w.wgu, nullptr, m->xs, w.sgu, nullptr, m->h, H, 2 * I, st))) return rc;
    fht_kernel<13, true><<<1, kFhtBlock, 0, st>>>(m->h, nullptr, m->xq, m->xs, c.fht_scale);
    if ((rc = launch_gemv<kEpiDequant>(m->xq, w.wd, nullptr, m->xs, w.sd, m->x2, m->x, I, H, st))) return rc;
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

static int decode_head(flexllm_llama* m, float* logits, hipStream_t st) {
    const flexllm_llama_config& c = m->cfg;
    rmsnorm_kernel<1, false, 512><<<1, 512, 0, st>>>(m->x, m->gamma + (size_t)(2 * c.layers) * c.hidden, m->nrm, nullptr,
                                                   nullptr, c.hidden, c.eps);
    return lm_head_launch(m->embed, m->nrm, logits, c.vocab, c.hidden, st);
}

// tokens_out != NULL: greedy mode, `steps` tokens in this launch (argmax, token hand-over and position advance inside the kernel)
static int launch_mega(flexllm_llama* m, int* token, const float* x_in, float* logits, int want_head, hipStream_t st,
                       int* tokens_out = nullptr, int steps = 1, const float* rands = nullptr, int top_k = 0) {
    const flexllm_llama_config& c = m->cfg;
    MegaParams p;
    p.layers = m->w4 ? (const void*)m->layers4_dev : (const void*)m->layers_dev;
    p.head_w4 = m->head_w4; p.head_s = m->head_s; p.head_sum = m->head_sum;
    p.gamma = m->gamma; p.q_s = m->q_s; p.k_s = m->k_s; p.v_s = m->v_s; p.a_s = m->a_s;
    p.rope_sin = m->rope_sin; p.rope_cos = m->rope_cos;
    p.embed = reinterpret_cast<const __half*>(m->embed);
    p.k_cache = m->k_cache; p.v_cache = m->v_cache; p.cache_layer_bytes = m->cache_layer_bytes;
    p.x = m->x; p.x2 = m->x2; p.qkv = m->qkv; p.h = m->h; p.logits = logits ? logits : m->logits;
    p.stats = m->stats; p.state = m->state;
    p.xarena = m->arena.base;
    for (int d = 0; d < 2; d++)
        for (int i = 0; i < 2; i++) p.xblk[d][i] = m->xblk[d][i];
    p.die_mask = m->arena.die_mask;
    p.token = token; p.tokens_out = tokens_out; p.n_steps = steps; p.x_in = x_in; p.am_v = m->am_v; p.am_i = m->am_i;
    p.n_layers = c.layers; p.max_pos = c.max_pos; p.vocab = c.vocab; p.want_head = want_head;
    p.top_k = top_k; p.rands = rands; p.cand_v = m->topk_val; p.cand_i = m->topk_idx;
    p.eps = c.eps; p.fht_scale = c.fht_scale;
    p.timeline = m->timeline;
    {   // debug aid: which workgroup's stamps to record (default 0)
        const char* e = getenv("FLEXLLM_TIMELINE_WG");
        const int w = e ? atoi(e) : 0;
        p.timeline_wg = w >= 0 && w < kMegaWG ? w : 0;
    }
    static std::atomic<bool> lds_opted_in{false};     // the kernels' LDS block exceeds the default 64 KiB per workgroup
    if (!lds_opted_in.load(std::memory_order_acquire)) {   // idempotent: two threads racing here both set the same attribute
        FX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(decode_mega_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)sizeof(MegaLds)));
        FX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(decode_mega_w4_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)sizeof(MegaLds)));
        lds_opted_in.store(true, std::memory_order_release);
    }
    // An ordinary launch: one workgroup per CU fits by construction (mega_ok checks the CU count), and every barrier
    // and poll in the kernel is bounded, so work of other streams that delays some workgroups costs time, not a hang.
    // (A cooperative launch gives the same timing, but rocprofv3 of this ROCm release crashes at exit after one.)
    if (m->w4) decode_mega_w4_kernel<<<kMegaWG, kMegaT, sizeof(MegaLds), st>>>(p);
    else decode_mega_kernel<<<kMegaWG, kMegaT, sizeof(MegaLds), st>>>(p);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

static inline bool use_mega(const flexllm_llama* m) { return m->mega_ok && m->decode_mode == 0; }

// One greedy step: embedding of *token_io -> layers -> head -> argmax -> *token_io, tokens_out[step], pos++.
static int greedy_step(flexllm_llama* m, int* token_io, int* tokens_out, hipStream_t st) {
    const flexllm_llama_config& c = m->cfg;
    embed_kernel<<<(c.hidden + 255) / 256, 256, 0, st>>>(reinterpret_cast<const __half*>(m->embed), token_io, m->x, c.hidden, c.vocab, &m->state[3]);
    int rc;
    for (int l = 0; l < c.layers; l++)
        if ((rc = decode_layer(m, l, st))) return rc;
    if ((rc = decode_head(m, m->logits, st))) return rc;
    argmax_partial_kernel<<<kArgmaxParts, 256, 0, st>>>(m->logits, c.vocab, m->am_v, m->am_i);
    argmax_final_advance_kernel<<<1, 64, 0, st>>>(m->am_v, m->am_i, kArgmaxParts, token_io, tokens_out, m->state);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx

using namespace fx;

extern "C" {

int flexllm_llama_create(flexllm_llama** out, const flexllm_llama_config* cfg, const flexllm_llama_weights* w) {
    FX_REQUIRE(out && cfg && w, "llama_create: null pointer");
    const flexllm_llama_config& c = *cfg;
    FX_REQUIRE(c.head_dim == kHd, "llama_create: head_dim=%d (only 64)", c.head_dim);
    FX_REQUIRE(c.layers > 0 && c.hidden == c.q_heads * c.head_dim && c.kv_hidden == c.kv_heads * c.head_dim,
               "llama_create: hidden=%d q_heads=%d kv_hidden=%d kv_heads=%d inconsistent", c.hidden, c.q_heads, c.kv_hidden, c.kv_heads);
    FX_REQUIRE(c.hidden == 2048 && c.inter == 8192, "llama_create: hidden=%d inter=%d (kernels are instantiated for 2048/8192)", c.hidden, c.inter);
    FX_REQUIRE(c.q_heads % c.kv_heads == 0 && c.q_heads / c.kv_heads <= 4, "llama_create: GQA group %d > 4", c.q_heads / c.kv_heads);
    FX_REQUIRE(c.max_pos > 0 && c.max_pos % kChunk == 0 && c.max_pos <= kChunk * kMaxChunks,
               "llama_create: max_pos=%d must be a multiple of 128, <= 8192", c.max_pos);
    FX_REQUIRE(c.vocab > 0, "llama_create: vocab=%d", c.vocab);
    flexllm_llama* m = new flexllm_llama();
    m->cfg = c;
    const int H = c.hidden, KV = c.kv_hidden, I = c.inter, L = c.layers;
    auto fail = [&](int rc) { flexllm_llama_destroy(m); return rc; };
#define FX_TRY(expr)                          \
    do {                                      \
        int rc__ = (expr);                    \
        if (rc__) return fail(rc__);          \
    } while (0)
#define FX_TRY_HIP(call)                                                               \
    do {                                                                               \
        hipError_t e_ = (call);                                                        \
        if (e_ != hipSuccess) {                                                        \
            set_error("%s failed: %s", #call, hipGetErrorString(e_));                  \
            return fail(FLEXLLM_EHIP);                                                 \
        }                                                                              \
    } while (0)
    m->layers.resize(L);
    for (int l = 0; l < L; l++) {
        LayerW& lw = m->layers[l];
        FX_TRY(dev_alloc(m, (void**)&lw.wqkv, (size_t)(H + 2 * KV) * H));
        FX_TRY(dev_alloc(m, (void**)&lw.wo, (size_t)H * H));
        FX_TRY(dev_alloc(m, (void**)&lw.wgu, (size_t)2 * I * H));
        FX_TRY(dev_alloc(m, (void**)&lw.wd, (size_t)H * I));
        FX_TRY(dev_alloc(m, (void**)&lw.sqkv, sizeof(float) * (H + 2 * KV)));
        FX_TRY(dev_alloc(m, (void**)&lw.so, sizeof(float) * H));
        FX_TRY(dev_alloc(m, (void**)&lw.sgu, sizeof(float) * 2 * I));
        FX_TRY(dev_alloc(m, (void**)&lw.sd, sizeof(float) * H));
        FX_TRY_HIP(hipMemcpy(lw.wqkv, w->wq[l], (size_t)H * H, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(lw.wqkv + (size_t)H * H, w->wk[l], (size_t)KV * H, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(lw.wqkv + (size_t)(H + KV) * H, w->wv[l], (size_t)KV * H, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(lw.wo, w->wo[l], (size_t)H * H, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy2D(lw.wgu, (size_t)2 * H, w->wg[l], H, H, I, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy2D(lw.wgu + H, (size_t)2 * H, w->wu[l], H, H, I, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(lw.wd, w->wd[l], (size_t)H * I, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(lw.sqkv, w->sq[l], sizeof(float) * H, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(lw.sqkv + H, w->sk[l], sizeof(float) * KV, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(lw.sqkv + H + KV, w->sv[l], sizeof(float) * KV, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(lw.so, w->so[l], sizeof(float) * H, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy2D(lw.sgu, 2 * sizeof(float), w->sg[l], sizeof(float), sizeof(float), I, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy2D(lw.sgu + 1, 2 * sizeof(float), w->su[l], sizeof(float), sizeof(float), I, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(lw.sd, w->sd[l], sizeof(float) * H, hipMemcpyDeviceToDevice));
    }
    auto dup = [&](void** dst, const void* src, size_t bytes) -> int {
        int rc = dev_alloc(m, dst, bytes);
        if (rc) return rc;
        hipError_t e = hipMemcpy(*dst, src, bytes, hipMemcpyDeviceToDevice);
        if (e != hipSuccess) { set_error("hipMemcpy failed: %s", hipGetErrorString(e)); return FLEXLLM_EHIP; }
        return FLEXLLM_OK;
    };
    FX_TRY(dup((void**)&m->gamma, w->gamma, sizeof(float) * (size_t)(2 * L + 1) * H));
    FX_TRY(dup((void**)&m->q_s, w->q_s, sizeof(float) * (size_t)L * c.q_heads));
    FX_TRY(dup((void**)&m->k_s, w->k_s, sizeof(float) * (size_t)L * c.kv_heads));
    FX_TRY(dup((void**)&m->v_s, w->v_s, sizeof(float) * (size_t)L * c.kv_heads));
    FX_TRY(dup((void**)&m->a_s, w->a_s, sizeof(float) * (size_t)L * c.q_heads));
    FX_TRY(dup((void**)&m->rope_sin, w->rope_sin, sizeof(float) * (size_t)c.max_pos * (kHd / 2)));
    FX_TRY(dup((void**)&m->rope_cos, w->rope_cos, sizeof(float) * (size_t)c.max_pos * (kHd / 2)));
    FX_TRY(dup((void**)&m->embed, w->embed, sizeof(uint16_t) * (size_t)c.vocab * H));
    m->cache_layer_bytes = (size_t)c.kv_heads * c.max_pos * kHd;
    FX_TRY(dev_alloc(m, (void**)&m->k_cache, m->cache_layer_bytes * L));
    FX_TRY(dev_alloc(m, (void**)&m->v_cache, m->cache_layer_bytes * L));
    FX_TRY_HIP(hipMemset(m->k_cache, 0, m->cache_layer_bytes * L));
    FX_TRY_HIP(hipMemset(m->v_cache, 0, m->cache_layer_bytes * L));
    FX_TRY(dev_alloc(m, (void**)&m->x, sizeof(float) * H));
    FX_TRY(dev_alloc(m, (void**)&m->x2, sizeof(float) * H));
    FX_TRY(dev_alloc(m, (void**)&m->nrm, sizeof(float) * H));
    FX_TRY(dev_alloc(m, (void**)&m->qkv, sizeof(float) * (H + 2 * KV)));
    FX_TRY(dev_alloc(m, (void**)&m->h, sizeof(float) * I * (size_t)kMegaMaxSteps * L));   // one slice per layer pass of a launch
    FX_TRY(dev_alloc(m, (void**)&m->logits, sizeof(float) * c.vocab));
    FX_TRY(dev_alloc(m, (void**)&m->xq, (size_t)I));
    FX_TRY(dev_alloc(m, (void**)&m->q8, (size_t)H));
    FX_TRY(dev_alloc(m, (void**)&m->xs, sizeof(float) * 4));
    FX_TRY(dev_alloc(m, (void**)&m->scores, sizeof(float) * (size_t)c.q_heads * c.max_pos));
    FX_TRY(dev_alloc(m, (void**)&m->stats, sizeof(float2) * (size_t)c.q_heads * kMaxChunks));
    FX_TRY(dev_alloc(m, (void**)&m->o_acc, sizeof(int32_t) * H));
    {
        // the exchange words of the persistent kernel: 11 blocks per die (FLEXLLM_DIE_COPIES=0: one copy, no calibration)
        const char* e = getenv("FLEXLLM_DIE_COPIES");
        void* raw = nullptr;
        const int rc_arena = die_arena_create(m->arena, 48, !(e && atoi(e) == 0), &raw);
        if (raw) m->owned.push_back(raw);
        FX_TRY(rc_arena);
        static_assert(sizeof(unsigned long long) * 1024 == kDieBlock && sizeof(int32_t) * 2048 == kDieBlock && sizeof(unsigned) * kMegaBarWords <= kDieBlock,
                      "the exchange arrays are cut into 8 KiB blocks");
        for (int k = 0; k < kXbCount; k++) {
            void* pr[2];
            if (!m->arena.take_pair(pr, k < kXbOacc ? 0xFF : 0)) { set_error("llama_create: the exchange arena is used up"); return fail(FLEXLLM_EHIP); }
            for (int d = 0; d < 2; d++) {
                m->xptr[d][k] = pr[d];
                const unsigned long long idx = (unsigned long long)((static_cast<char*>(pr[d]) - m->arena.base) / kDieBlock);
                m->xblk[d][k / 8] |= idx << (8 * (k % 8));
            }
        }
    }
    FX_TRY(dev_alloc(m, (void**)&m->state, sizeof(int) * 8));
    FX_TRY(dev_alloc(m, (void**)&m->am_v, sizeof(float) * kArgmaxParts));
    // per-workgroup sampling candidates: of the persistent kernel's workgroups or of the stand-alone first stage
    constexpr int kCandGroups = kMegaWG > kTopKParts ? kMegaWG : kTopKParts;
    FX_TRY(dev_alloc(m, (void**)&m->topk_val, sizeof(float) * kCandGroups * kTopKMax));
    FX_TRY(dev_alloc(m, (void**)&m->topk_idx, sizeof(int) * kCandGroups * kTopKMax));
    FX_TRY(dev_alloc(m, (void**)&m->am_i, sizeof(int) * kArgmaxParts));
    FX_TRY(dev_alloc(m, (void**)&m->layers_dev, sizeof(LayerW) * L));
    FX_TRY_HIP(hipMemcpy(m->layers_dev, m->layers.data(), sizeof(LayerW) * L, hipMemcpyHostToDevice));
    FX_TRY_HIP(hipMemset(m->state, 0, sizeof(int) * 8));
    FX_TRY_HIP(hipMemset(m->o_acc, 0, sizeof(int32_t) * H));
    FX_TRY_HIP(hipMemset(m->am_v, 0, sizeof(float) * kArgmaxParts));
    FX_TRY_HIP(hipMemset(m->am_i, 0, sizeof(int) * kArgmaxParts));
    FX_TRY_HIP(hipMemset(m->topk_val, 0, sizeof(float) * kCandGroups * kTopKMax));
    FX_TRY_HIP(hipMemset(m->topk_idx, 0, sizeof(int) * kCandGroups * kTopKMax));
    {
        int dev = 0, cus = 0;
        FX_TRY_HIP(hipGetDevice(&dev));
        FX_TRY_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        // the persistent kernel needs all its workgroups resident at once and is compiled for these shapes
        m->mega_ok = cus >= kMegaWG && c.hidden == 2048 && c.kv_hidden == 512 && c.inter == 8192 && c.q_heads == 32 &&
                     c.kv_heads == 8 && c.max_pos <= 32 * kChunk && kArgmaxParts >= kMegaWG;
    }
    FX_TRY_HIP(hipDeviceSynchronize());
#undef FX_TRY
#undef FX_TRY_HIP
    *out = m;
    return FLEXLLM_OK;
}

int flexllm_llama_create_w4a4(flexllm_llama** out, const flexllm_llama_config* cfg, const flexllm_llama_w4a4_weights* w) {
    FX_REQUIRE(out && cfg && w, "llama_create_w4a4: null pointer");
    FX_REQUIRE(w->sumq && w->sumk && w->sumv && w->sumo && w->sumg && w->sumu && w->sumd && w->head_w && w->head_s && w->head_sum,
               "llama_create_w4a4: null weight pointer");
    // The common part (fused q/k/v rows, interleaved gate/up rows, scales, tables, caches, workspace) is that of the
    // W8A8 model on the same values held one per byte; the matrices are then packed two values per byte.
    flexllm_llama* m = nullptr;
    int rc = flexllm_llama_create(&m, cfg, &w->base);
    if (rc) return rc;
    const flexllm_llama_config& c = m->cfg;
    const int H = c.hidden, KV = c.kv_hidden, I = c.inter, L = c.layers;
    auto fail = [&](int code) { flexllm_llama_destroy(m); return code; };
    if (!m->mega_ok) {
        set_error("llama_create_w4a4: the W4A4 decode path is the persistent kernel only (needs >= %d CUs and Llama-3.2-1B shapes)", kMegaWG);
        return fail(FLEXLLM_EINVAL);
    }
#define FX_TRY(expr)                          \
    do {                                      \
        int rc__ = (expr);                    \
        if (rc__) return fail(rc__);          \
    } while (0)
#define FX_TRY_HIP(call)                                                               \
    do {                                                                               \
        hipError_t e_ = (call);                                                        \
        if (e_ != hipSuccess) {                                                        \
            set_error("%s failed: %s", #call, hipGetErrorString(e_));                  \
            return fail(FLEXLLM_EHIP);                                                 \
        }                                                                              \
    } while (0)
    // Every matrix must hold 4-bit values: the prefill graph multiplies the bytes as they are, the persistent decode
    // kernel their low nibbles, and the two would silently part on anything outside -8..7.
    unsigned* bad = reinterpret_cast<unsigned*>(m->state) + 7;     // a word of the token state no kernel uses at create time
    FX_TRY_HIP(hipMemset(bad, 0, sizeof(unsigned)));
    auto pack = [&](const int8_t* values, int8_t** packed, size_t n_values) -> int {
        int r = dev_alloc(m, (void**)packed, n_values / 2);
        if (r) return r;
        const size_t n_out = n_values / 2;
        nibble_range_kernel<<<(int)((n_values + 255) / 256 < 4096 ? (n_values + 255) / 256 : 4096), 256>>>(values, n_values, bad);
        pack_nibbles_kernel<<<(int)((n_out + 255) / 256 < 4096 ? (n_out + 255) / 256 : 4096), 256>>>(
            reinterpret_cast<const uint8_t*>(values), reinterpret_cast<uint8_t*>(*packed), n_out);
        return FLEXLLM_OK;
    };
    m->layers4.resize(L);
    for (int l = 0; l < L; l++) {
        const LayerW& lw = m->layers[l];
        LayerW4& l4 = m->layers4[l];
        FX_TRY(pack(lw.wqkv, &l4.wqkv, (size_t)(H + 2 * KV) * H));
        FX_TRY(pack(lw.wo, &l4.wo, (size_t)H * H));
        FX_TRY(pack(lw.wgu, &l4.wgu, (size_t)2 * I * H));
        FX_TRY(pack(lw.wd, &l4.wd, (size_t)H * I));
        l4.sqkv = lw.sqkv; l4.so = lw.so; l4.sgu = lw.sgu; l4.sd = lw.sd;
        FX_TRY(dev_alloc(m, (void**)&l4.mqkv, sizeof(float) * (H + 2 * KV)));
        FX_TRY(dev_alloc(m, (void**)&l4.mo, sizeof(float) * H));
        FX_TRY(dev_alloc(m, (void**)&l4.mgu, sizeof(float) * 2 * I));
        FX_TRY(dev_alloc(m, (void**)&l4.md, sizeof(float) * H));
        FX_TRY_HIP(hipMemcpy(l4.mqkv, w->sumq[l], sizeof(float) * H, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(l4.mqkv + H, w->sumk[l], sizeof(float) * KV, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(l4.mqkv + H + KV, w->sumv[l], sizeof(float) * KV, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(l4.mo, w->sumo[l], sizeof(float) * H, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy2D(l4.mgu, 2 * sizeof(float), w->sumg[l], sizeof(float), sizeof(float), I, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy2D(l4.mgu + 1, 2 * sizeof(float), w->sumu[l], sizeof(float), sizeof(float), I, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(l4.md, w->sumd[l], sizeof(float) * H, hipMemcpyDeviceToDevice));
    }
    {
        int8_t* hw = nullptr;
        FX_TRY(pack(w->head_w, &hw, (size_t)c.vocab * H));
        m->head_w4 = reinterpret_cast<uint8_t*>(hw);
        FX_TRY(dev_alloc(m, (void**)&m->head_s, sizeof(float) * c.vocab));
        FX_TRY(dev_alloc(m, (void**)&m->head_sum, sizeof(float) * c.vocab));
        FX_TRY_HIP(hipMemcpy(m->head_s, w->head_s, sizeof(float) * c.vocab, hipMemcpyDeviceToDevice));
        FX_TRY_HIP(hipMemcpy(m->head_sum, w->head_sum, sizeof(float) * c.vocab, hipMemcpyDeviceToDevice));
    }
    FX_TRY(dev_alloc(m, (void**)&m->layers4_dev, sizeof(LayerW4) * L));
    FX_TRY_HIP(hipMemcpy(m->layers4_dev, m->layers4.data(), sizeof(LayerW4) * L, hipMemcpyHostToDevice));
    FX_TRY_HIP(hipDeviceSynchronize());
    FX_TRY_HIP(hipGetLastError());
    {
        unsigned n_bad = 0;
        FX_TRY_HIP(hipMemcpy(&n_bad, bad, sizeof(unsigned), hipMemcpyDeviceToHost));
        FX_TRY_HIP(hipMemset(bad, 0, sizeof(unsigned)));
        if (n_bad) {
            set_error("llama_create_w4a4: %u weight values lie outside -8..7 (not a 4-bit export)", n_bad);
            return fail(FLEXLLM_EINVAL);
        }
    }
#undef FX_TRY
#undef FX_TRY_HIP
    m->w4 = true;
    *out = m;
    return FLEXLLM_OK;
}

int flexllm_llama_destroy(flexllm_llama* m) {
    if (!m) return FLEXLLM_OK;
    (void)hipDeviceSynchronize();
    if (m->graph_exec) (void)hipGraphExecDestroy(m->graph_exec);
    prefill_workspace_destroy(&m->pws);
    for (void* p : m->owned) (void)hipFree(p);
    delete m;
    return FLEXLLM_OK;
}

int flexllm_llama_set_decode_mode(flexllm_llama* m, int mode) {
    FX_REQUIRE(m && (mode == 0 || mode == 1), "llama_set_decode_mode: mode=%d (0 persistent kernel, 1 one kernel per stage)", mode);
    FX_REQUIRE(!(m->w4 && mode == 1), "llama_set_decode_mode: a W4A4 model decodes with the persistent kernel only");
    if (m->decode_mode != mode) {
        if (m->graph_exec) { (void)hipGraphExecDestroy(m->graph_exec); m->graph_exec = nullptr; }
        // (the two schedules keep their attention accumulators apart: the persistent kernel's are back at zero
        // whenever it ends, the per-stage kernels clear theirs before use)
    }
    m->decode_mode = mode;
    return FLEXLLM_OK;
}

int flexllm_die_classify(const float* us, int n_blocks, int* usable, unsigned* die_mask, int* die_of_block, float* near_us, float* far_us) {
    FX_REQUIRE(us && usable && die_mask && die_of_block && near_us && far_us && n_blocks > 0, "die_classify: bad arguments");
    *die_mask = 0; *near_us = 0.0f; *far_us = 0.0f;
    for (int b = 0; b < n_blocks; b++) die_of_block[b] = -1;
    *usable = die_classify(us, n_blocks, die_mask, die_of_block, near_us, far_us) ? 1 : 0;
    return FLEXLLM_OK;
}

int flexllm_llama_exchange_info(const flexllm_llama* m, int* two_copies, unsigned* die_mask, float* near_us, float* far_us) {
    FX_REQUIRE(m && two_copies && die_mask && near_us && far_us, "llama_exchange_info: null pointer");
    *two_copies = m->arena.calibrated ? 1 : 0;
    *die_mask = m->arena.die_mask;
    *near_us = m->arena.near_us;
    *far_us = m->arena.far_us;
    return FLEXLLM_OK;
}

int flexllm_llama_stage_timeline(flexllm_llama* m, long long* host_out, int max_entries) {
    FX_REQUIRE(m && host_out && max_entries > 0, "llama_stage_timeline: bad arguments");
    // stage stamps, fine stamps, per-workgroup entry and exit, one layer's stamps of every workgroup (debug builds)
    const int n = m->cfg.layers * 12 + 2 + 64 + 2 * fx::kMegaWG + 12 * fx::kMegaWG;
    if (!m->timeline) {
        int rc = dev_alloc(m, (void**)&m->timeline, sizeof(long long) * n);
        if (rc) return rc;
        FX_HIP(hipMemset(m->timeline, 0, sizeof(long long) * n));
        if (m->graph_exec) { (void)hipGraphExecDestroy(m->graph_exec); m->graph_exec = nullptr; }
        for (int i = 0; i < max_entries; i++) host_out[i] = 0;
        return FLEXLLM_OK;
    }
    FX_HIP(hipDeviceSynchronize());
    FX_HIP(hipMemcpy(host_out, m->timeline, sizeof(long long) * (n < max_entries ? n : max_entries), hipMemcpyDeviceToHost));
    return FLEXLLM_OK;
}

int flexllm_llama_check(flexllm_llama* m) {
    FX_REQUIRE(m, "llama_check: null pointer");
    FX_HIP(hipDeviceSynchronize());
    int st[4] = {0, 0, 0, 0};
    FX_HIP(hipMemcpy(st, m->state, sizeof(st), hipMemcpyDeviceToHost));
    if (st[3] != 0) {
        (void)hipMemset(&m->state[3], 0, sizeof(int));
        if (st[3] == 2) {
            set_error("decode: a token id outside the vocabulary (%d entries) was fed in; token 0 was used instead", m->cfg.vocab);
            return FLEXLLM_EINVAL;
        }
        // after a time-out the barrier counters and the attention accumulators hold partial counts: start them afresh
        for (int d = 0; d < 2; d++) (void)hipMemset(m->xptr[d][kXbBar], 0, kDieBlock);
        (void)hipMemset(&m->state[2], 0, sizeof(int));
        for (int d = 0; d < 2; d++) (void)hipMemset(m->xptr[d][kXbOacc], 0, kDieBlock);
        set_error("persistent decode kernel: a wait timed out (were all %d workgroups resident?)", kMegaWG);
        return FLEXLLM_EHIP;
    }
    return FLEXLLM_OK;
}

int flexllm_llama_kv_cache(flexllm_llama* m, int8_t** k_cache, int8_t** v_cache) {
    FX_REQUIRE(m && k_cache && v_cache, "llama_kv_cache: null pointer");
    *k_cache = m->k_cache;
    *v_cache = m->v_cache;
    return FLEXLLM_OK;
}

int flexllm_llama_decode_hidden(flexllm_llama* m, const float* x_in, int pos, float* hidden_out, float* logits,
                                void* stream) {
    FX_REQUIRE(m && x_in, "llama_decode_hidden: null pointer");
    FX_REQUIRE(pos >= 0 && pos < m->cfg.max_pos, "llama_decode_hidden: pos=%d outside [0,%d)", pos, m->cfg.max_pos);
    hipStream_t st = as_stream(stream);
    const int H = m->cfg.hidden;
    set_state_kernel<<<1, 1, 0, st>>>(m->state, pos, 0);
    if (use_mega(m)) {
        int rc = launch_mega(m, nullptr, x_in, logits, logits != nullptr, st);
        if (rc) return rc;
        if (hidden_out) FX_HIP(hipMemcpyAsync(hidden_out, m->x, sizeof(float) * H, hipMemcpyDeviceToDevice, st));
        return FLEXLLM_OK;
    }
    FX_HIP(hipMemcpyAsync(m->x, x_in, sizeof(float) * H, hipMemcpyDeviceToDevice, st));
    for (int l = 0; l < m->cfg.layers; l++) {
        int rc = decode_layer(m, l, st);
        if (rc) return rc;
    }
    if (hidden_out) FX_HIP(hipMemcpyAsync(hidden_out, m->x, sizeof(float) * H, hipMemcpyDeviceToDevice, st));
    if (logits) {
        int rc = decode_head(m, logits, st);
        if (rc) return rc;
    }
    return FLEXLLM_OK;
}

int flexllm_llama_decode_greedy(flexllm_llama* m, int* token_io, int pos0, int steps, int* tokens_out, int use_graph,
                                void* stream) {
    FX_REQUIRE(m && token_io && tokens_out, "llama_decode_greedy: null pointer");
    FX_REQUIRE(steps >= 0 && pos0 >= 0 && pos0 + steps <= m->cfg.max_pos,
               "llama_decode_greedy: pos0=%d steps=%d exceed max_pos=%d", pos0, steps, m->cfg.max_pos);
    hipStream_t st = as_stream(stream);
    set_state_kernel<<<1, 1, 0, st>>>(m->state, pos0, 0);
    FX_LAUNCH_CHECK();
    if (use_mega(m)) {
        // the persistent kernel generates up to kMegaMaxSteps tokens per launch; a graph would have nothing to add
        for (int s = 0; s < steps; s += kMegaMaxSteps) {
            int rc = launch_mega(m, token_io, nullptr, nullptr, 1, st, tokens_out, steps - s < kMegaMaxSteps ? steps - s : kMegaMaxSteps);
            if (rc) return rc;
        }
        return FLEXLLM_OK;
    }
    if (!use_graph) {
        for (int s = 0; s < steps; s++) {
            int rc = greedy_step(m, token_io, tokens_out, st);
            if (rc) return rc;
        }
        return FLEXLLM_OK;
    }
    FX_REQUIRE(st != nullptr, "llama_decode_greedy: graph replay needs a non-default stream");
    if (!m->graph_exec || m->graph_token_io != token_io || m->graph_tokens_out != tokens_out || m->graph_stream != st) {
        if (m->graph_exec) { (void)hipGraphExecDestroy(m->graph_exec); m->graph_exec = nullptr; }
        FX_HIP(hipStreamSynchronize(st));
        hipGraph_t graph;
        FX_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        int rc = greedy_step(m, token_io, tokens_out, st);
        hipError_t e = hipStreamEndCapture(st, &graph);
        if (rc) { if (e == hipSuccess) (void)hipGraphDestroy(graph); return rc; }
        FX_HIP(e);
        e = hipGraphInstantiate(&m->graph_exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        FX_HIP(e);
        m->graph_token_io = token_io;
        m->graph_tokens_out = tokens_out;
        m->graph_stream = st;
    }
    for (int s = 0; s < steps; s++) FX_HIP(hipGraphLaunch(m->graph_exec, st));
    return FLEXLLM_OK;
}

int flexllm_llama_decode_sample(flexllm_llama* m, int* token_io, int pos0, int steps, const float* rands, int top_k,
                                int* tokens_out, void* stream) {
    FX_REQUIRE(m && token_io && tokens_out && rands, "llama_decode_sample: null pointer");
    FX_REQUIRE(steps >= 0 && pos0 >= 0 && pos0 + steps <= m->cfg.max_pos,
               "llama_decode_sample: pos0=%d steps=%d exceed max_pos=%d", pos0, steps, m->cfg.max_pos);
    FX_REQUIRE(top_k >= 1 && top_k <= kTopKMax && top_k <= m->cfg.vocab, "llama_decode_sample: top_k=%d (1..%d)", top_k, kTopKMax);
    hipStream_t st = as_stream(stream);
    const flexllm_llama_config& c = m->cfg;
    set_state_kernel<<<1, 1, 0, st>>>(m->state, pos0, 0);
    FX_LAUNCH_CHECK();
    if (use_mega(m) && (c.vocab + kMegaWG - 1) / kMegaWG <= 4096) {
        // the persistent kernel samples by itself (per-workgroup candidates, one more grid barrier, every workgroup
        // draws the same token): up to kMegaMaxSteps tokens per launch, as in greedy mode
        for (int s = 0; s < steps; s += kMegaMaxSteps) {
            int rc = launch_mega(m, token_io, nullptr, nullptr, 1, st, tokens_out, steps - s < kMegaMaxSteps ? steps - s : kMegaMaxSteps,
                                 rands, top_k);
            if (rc) return rc;
        }
        return FLEXLLM_OK;
    }
    FX_REQUIRE(!m->w4, "llama_decode_sample: vocab=%d is too large for the persistent kernel's sampler, the only one a W4A4 model has", c.vocab);
    // one kernel per stage: layers + lm_head into m->logits, then the sampler picks the token (rands[step]), hands it
    // over through token_io and advances position and step in device memory
    TopKOut out = {nullptr, nullptr, nullptr, nullptr, token_io, tokens_out, m->state};
    for (int s = 0; s < steps; s++) {
        int rc;
        embed_kernel<<<(c.hidden + 255) / 256, 256, 0, st>>>(reinterpret_cast<const __half*>(m->embed), token_io, m->x, c.hidden, c.vocab, &m->state[3]);
        for (int l = 0; l < c.layers; l++)
            if ((rc = decode_layer(m, l, st))) return rc;
        if ((rc = decode_head(m, m->logits, st))) return rc;
        // two stages: 128 workgroups pick the top_k of their share of the vocabulary, one workgroup picks among those
        topk_partial_kernel<<<kTopKParts, kTopKPartThreads, 0, st>>>(m->logits, c.vocab, top_k, m->topk_val, m->topk_idx);
        topk_sample_kernel<256><<<1, 256, 0, st>>>(m->topk_val, m->topk_idx, kTopKParts * top_k, top_k, rands, 1, 1, out);
        FX_LAUNCH_CHECK();
    }
    return FLEXLLM_OK;
}

int flexllm_llama_generate(flexllm_llama* m, const int* prompt, int n_prompt, int steps, const float* rands, int top_k,
                           int* tokens_out, void* stream) {
    FX_REQUIRE(m && prompt && tokens_out, "llama_generate: null pointer");
    FX_REQUIRE(n_prompt >= 1 && steps >= 0 && n_prompt - 1 + steps <= m->cfg.max_pos,
               "llama_generate: prompt of %d tokens + %d steps exceed max_pos=%d", n_prompt, steps, m->cfg.max_pos);
    FX_REQUIRE(top_k == 0 || rands, "llama_generate: sampling (top_k=%d) needs the uniform numbers", top_k);
    hipStream_t st = as_stream(stream);
    const flexllm_llama_config& c = m->cfg;
    const int s = n_prompt - 1;                               // prefilled tokens: all but the last one
    const int rows = (s + 31) / 32 * 32;                      // the prefill works on tiles of 32 rows
    FX_REQUIRE(rows <= c.max_pos, "llama_generate: %d prompt rows (padded to 32) exceed max_pos=%d", rows, c.max_pos);
    if (!m->gen_token) FX_ALLOC(m, m->gen_token, sizeof(int));
    if (rows > 0) {
        if (!m->gen_x) {                                      // once, for the longest prompt the cache admits
            m->gen_rows = (c.max_pos + 31) / 32 * 32;
            FX_ALLOC(m, m->gen_x, sizeof(float) * (size_t)m->gen_rows * c.hidden);
        }
        embed_rows_kernel<<<rows, 256, 0, st>>>(reinterpret_cast<const __half*>(m->embed), prompt, s, m->gen_x, c.hidden, c.vocab,
                                                &m->state[3]);
        FX_LAUNCH_CHECK();
        // rows s..rows-1 are zero padding: they write cache rows at positions >= s, which the decode steps below
        // overwrite one by one before any of them is read
        int rc = m->w4 ? llama_prefill_run_w4a4(c, m->layers.data(), m->layers4.data(), m->gamma, m->q_s, m->k_s, m->v_s, m->a_s,
                                                m->rope_sin, m->rope_cos, m->k_cache, m->v_cache, m->cache_layer_bytes,
                                                &m->pws, m->gen_x, rows, nullptr, st)
                       : llama_prefill_run(c, m->layers.data(), m->gamma, m->q_s, m->k_s, m->v_s, m->a_s, m->rope_sin, m->rope_cos,
                                           m->k_cache, m->v_cache, m->cache_layer_bytes, &m->pws, m->gen_x, rows, nullptr, st);
        if (rc) return rc;
    }
    copy_int_kernel<<<1, 1, 0, st>>>(prompt + s, m->gen_token);
    FX_LAUNCH_CHECK();
    if (steps == 0) return FLEXLLM_OK;
    if (top_k == 0) return flexllm_llama_decode_greedy(m, m->gen_token, s, steps, tokens_out, 0, stream);
    return flexllm_llama_decode_sample(m, m->gen_token, s, steps, rands, top_k, tokens_out, stream);
}

int flexllm_llama_prefill_hidden(flexllm_llama* m, const float* x_in, int s, float* hidden_out, void* stream) {
    FX_REQUIRE(m && x_in, "llama_prefill_hidden: null pointer");
    if (m->w4)
        return llama_prefill_run_w4a4(m->cfg, m->layers.data(), m->layers4.data(), m->gamma, m->q_s, m->k_s, m->v_s, m->a_s,
                                      m->rope_sin, m->rope_cos, m->k_cache, m->v_cache, m->cache_layer_bytes, &m->pws, x_in, s,
                                      hidden_out, as_stream(stream));
    return llama_prefill_run(m->cfg, m->layers.data(), m->gamma, m->q_s, m->k_s, m->v_s, m->a_s, m->rope_sin, m->rope_cos,
                             m->k_cache, m->v_cache, m->cache_layer_bytes, &m->pws, x_in, s, hidden_out, as_stream(stream));
}

}  // extern "C"

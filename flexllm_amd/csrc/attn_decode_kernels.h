// Decode attention over the int8 KV cache (one query token, GQA), and the cache append.
//
// Cache layout of one layer (head-major so that a head's keys are contiguous in HBM):
//   K: [kv_head][pos][64]                int8   - 64 B per key, a 128-key chunk is one 8 KiB burst
//   V: [kv_head][pos/64][64 ch][64 pos]  int8   - transposed in 64-position blocks so that P.V is a
//                                                 dot product along contiguous bytes (v_dot4_i32_i8)
// The reference rounds the probabilities to uint8 AFTER normalising by the full-row sum, so an online
// softmax that rescales at the end would round differently.  Three phases instead:
//   A  scores: one workgroup per (kv head, 128-key chunk); int32 q.k -> fp32 score, chunk max and
//      chunk sum of exp written beside the scores (L2-resident scratch)
//   B  one workgroup per (kv head, chunk): combine the chunk statistics into the row max / row sum,
//      p = exp(s-max)*(1/sum), P = min(255, round(p/A_s)), partial P.V in int32, atomically added
//      (integer adds: exact in any order)
//   C  dequantise the 32x64 int32 result.
// P is unsigned and V signed; gfx950's v_dot4_i32_i8 is signed x signed, so P.V is evaluated as
// (P-128).V + 128*sum(V), both exact.
#pragma once
#include "common.h"
#include <mutex>

namespace fx {

constexpr int kHd = 64;          // head_dim
constexpr int kChunk = 128;      // keys per workgroup
constexpr int kMaxChunks = 64;   // len <= 8192
constexpr int kVBlock = 64;      // positions per transposed V block

__device__ __forceinline__ size_t k_index(int kvh, int pos, int max_pos) { return ((size_t)kvh * max_pos + pos) * kHd; }
__device__ __forceinline__ size_t v_index(int kvh, int pos, int d, int max_pos) {
    return (((size_t)kvh * (max_pos / kVBlock) + pos / kVBlock) * kHd + d) * kVBlock + pos % kVBlock;
}

__device__ __forceinline__ int static_q8(float x, float div) {
    int r = (int)roundf(x / div);
    return r > 127 ? 127 : r < -128 ? -128 : r;
}

// k, v fp32 [tokens][kv_heads][64] -> caches at positions pos0..pos0+tokens-1
static __global__ __launch_bounds__(256) void kv_append_kernel(const float* __restrict__ k, const float* __restrict__ v,
                                                        int8_t* __restrict__ kc, int8_t* __restrict__ vc,
                                                        const float* __restrict__ k_s, const float* __restrict__ v_s,
                                                        int tokens, int kv_heads, int max_pos, int pos0) {
    const size_t n = (size_t)tokens * kv_heads * kHd;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const int d = (int)(i % kHd);
        const int h = (int)((i / kHd) % kv_heads);
        const int t = (int)(i / ((size_t)kHd * kv_heads));
        kc[k_index(h, pos0 + t, max_pos) + d] = (int8_t)static_q8(k[i], 1.0f * k_s[h]);
        vc[v_index(h, pos0 + t, d, max_pos)] = (int8_t)static_q8(v[i], 1.0f * v_s[h]);
    }
}

// int8 [tokens][kv_heads][64] already quantised -> cache layouts (used by prefill and by tests)
static __global__ __launch_bounds__(256) void kv_store_kernel(const int8_t* __restrict__ k8, const int8_t* __restrict__ v8,
                                                       int8_t* __restrict__ kc, int8_t* __restrict__ vc, int tokens,
                                                       int kv_heads, int max_pos, int pos0) {
    const size_t n = (size_t)tokens * kv_heads * kHd;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const int d = (int)(i % kHd);
        const int h = (int)((i / kHd) % kv_heads);
        const int t = (int)(i / ((size_t)kHd * kv_heads));
        kc[k_index(h, pos0 + t, max_pos) + d] = k8[i];
        vc[v_index(h, pos0 + t, d, max_pos)] = v8[i];
    }
}

// RoPE on q and k, static int8 quantisation of q/k/v, append of k/v to the cache.  One block per token:
// qkv is fp32 [tokens][H + 2*KV] = [q | k | v]; token t sits at position state[0] (decode, device-side
// position) or pos0 + t (prefill).  q8 is [tokens][H].
static __global__ __launch_bounds__(256) void qkv_post_kernel(const float* __restrict__ qkv_all, const float* __restrict__ sin_t,
                                                              const float* __restrict__ cos_t, const float* __restrict__ q_s,
                                                              const float* __restrict__ k_s, const float* __restrict__ v_s,
                                                              int8_t* __restrict__ q8_all, int8_t* __restrict__ kc,
                                                              int8_t* __restrict__ vc, const int* __restrict__ state, int pos0,
                                                              int q_heads, int kv_heads, int max_pos) {
    const int pos = state ? state[0] : pos0 + (int)blockIdx.x;
    const int half = kHd / 2;
    const float* sn = sin_t + (size_t)pos * half;
    const float* cs = cos_t + (size_t)pos * half;
    const int H = q_heads * kHd, KV = kv_heads * kHd;
    const float* qkv = qkv_all + (size_t)blockIdx.x * (H + 2 * KV);
    int8_t* q8 = q8_all + (size_t)blockIdx.x * H;
    const int q_pairs = q_heads * half, k_pairs = kv_heads * half;
    for (int i = threadIdx.x; i < q_pairs + k_pairs + KV; i += 256) {
        if (i < q_pairs) {
            const int hd = i / half, k = i % half;
            const float t0 = qkv[hd * kHd + k], t1 = qkv[hd * kHd + k + half];
            const float o0 = t0 * cs[k] - t1 * sn[k];
            const float o1 = t0 * sn[k] + t1 * cs[k];
            const float div = 8.0f * q_s[hd];      // sqrt(head_dim) folded into the Q scale
            q8[hd * kHd + k] = (int8_t)static_q8(o0, div);
            q8[hd * kHd + k + half] = (int8_t)static_q8(o1, div);
        } else if (i < q_pairs + k_pairs) {
            const int j = i - q_pairs;
            const int hd = j / half, k = j % half;
            const float t0 = qkv[H + hd * kHd + k], t1 = qkv[H + hd * kHd + k + half];
            const float o0 = t0 * cs[k] - t1 * sn[k];
            const float o1 = t0 * sn[k] + t1 * cs[k];
            const float div = 1.0f * k_s[hd];
            int8_t* dst = kc + k_index(hd, pos, max_pos);
            dst[k] = (int8_t)static_q8(o0, div);
            dst[k + half] = (int8_t)static_q8(o1, div);
        } else {
            const int j = i - q_pairs - k_pairs;
            const int hd = j / kHd, d = j % kHd;
            vc[v_index(hd, pos, d, max_pos)] = (int8_t)static_q8(qkv[H + KV + j], 1.0f * v_s[hd]);
        }
    }
}

// ---- phase A ------------------------------------------------------------------------------
// grid (nchunks, kv_heads); block 64*group threads: wave g = query head kvh*group+g, lane = key.
static __global__ __launch_bounds__(256) void dec_scores_kernel(const int8_t* __restrict__ q8, const int8_t* __restrict__ kc,
                                                         const float* __restrict__ q_s, const float* __restrict__ k_s,
                                                         float* __restrict__ scores, float2* __restrict__ stats,
                                                         int32_t* __restrict__ o_acc, const int* __restrict__ pos_ptr,
                                                         int len, int ld, int group, int max_pos) {
    // pos_ptr != NULL: the sequence length lives in device memory (position of the newest token + 1), so
    // that a captured graph can be replayed as the context grows; the grid then covers max_pos.
    if (pos_ptr) len = pos_ptr[0] + 1;
    const int chunk = blockIdx.x, kvh = blockIdx.y;
    if (chunk * kChunk >= len) return;
    const int g = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int qh = kvh * group + g;
    if (chunk == 0) o_acc[qh * kHd + lane] = 0;   // cleared here, accumulated in phase B
    const i32x4* qv = reinterpret_cast<const i32x4*>(q8 + (size_t)qh * kHd);
    const i32x4 q0 = qv[0], q1 = qv[1], q2 = qv[2], q3 = qv[3];
    const float sq = q_s[qh], sk = k_s[kvh];
    float sc[kChunk / 64];
    float mx = -1e32f;
#pragma unroll
    for (int j = 0; j < kChunk / 64; j++) {
        const int pos = chunk * kChunk + j * 64 + lane;
        sc[j] = -1e32f;
        if (pos < len) {
            const i32x4* kr = reinterpret_cast<const i32x4*>(kc + k_index(kvh, pos, max_pos));
            const i32x4 a = kr[0], b = kr[1], c = kr[2], d = kr[3];
            int acc = 0;
            acc = __builtin_amdgcn_sdot4(a.x, q0.x, acc, false); acc = __builtin_amdgcn_sdot4(a.y, q0.y, acc, false);
            acc = __builtin_amdgcn_sdot4(a.z, q0.z, acc, false); acc = __builtin_amdgcn_sdot4(a.w, q0.w, acc, false);
            acc = __builtin_amdgcn_sdot4(b.x, q1.x, acc, false); acc = __builtin_amdgcn_sdot4(b.y, q1.y, acc, false);
            acc = __builtin_amdgcn_sdot4(b.z, q1.z, acc, false); acc = __builtin_amdgcn_sdot4(b.w, q1.w, acc, false);
            acc = __builtin_amdgcn_sdot4(c.x, q2.x, acc, false); acc = __builtin_amdgcn_sdot4(c.y, q2.y, acc, false);
            acc = __builtin_amdgcn_sdot4(c.z, q2.z, acc, false); acc = __builtin_amdgcn_sdot4(c.w, q2.w, acc, false);
            acc = __builtin_amdgcn_sdot4(d.x, q3.x, acc, false); acc = __builtin_amdgcn_sdot4(d.y, q3.y, acc, false);
            acc = __builtin_amdgcn_sdot4(d.z, q3.z, acc, false); acc = __builtin_amdgcn_sdot4(d.w, q3.w, acc, false);
            sc[j] = (float)acc * sq * sk;
            scores[(size_t)qh * ld + pos] = sc[j];
            mx = fmaxf(mx, sc[j]);
        }
    }
    mx = wave_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < kChunk / 64; j++)
        if (chunk * kChunk + j * 64 + lane < len) sum += exp_f(sc[j] - mx);
    sum = wave_sum(sum);
    if (lane == 0) stats[qh * kMaxChunks + chunk] = make_float2(mx, sum);
}

// ---- phase B ------------------------------------------------------------------------------
static __global__ __launch_bounds__(256) void dec_pv_kernel(const float* __restrict__ scores, const float2* __restrict__ stats,
                                                     const int8_t* __restrict__ vc, const float* __restrict__ a_s,
                                                     int32_t* __restrict__ o_acc, uint8_t* __restrict__ p8_out,
                                                     const int* __restrict__ pos_ptr, int len, int ld, int group,
                                                     int max_pos) {
    __shared__ uint32_t p_lds[4][kChunk / 4];   // (P-128) bytes, per wave
    if (pos_ptr) len = pos_ptr[0] + 1;
    const int nchunks = (len + kChunk - 1) / kChunk;
    const int chunk = blockIdx.x, kvh = blockIdx.y;
    if (chunk * kChunk >= len) return;
    const int g = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int qh = kvh * group + g;
    // row statistics from the chunk statistics
    float m_c = -1e32f, l_c = 0.0f;
    if (lane < nchunks) { const float2 st = stats[qh * kMaxChunks + lane]; m_c = st.x; l_c = st.y; }
    const float mx = wave_max(m_c);
    const float sum = wave_sum(lane < nchunks ? l_c * exp_f(m_c - mx) : 0.0f);
    const float cd = 1.0f / sum;
    const float as = 1.0f * a_s[qh];
    uint8_t* pb = reinterpret_cast<uint8_t*>(p_lds[g]);
#pragma unroll
    for (int j = 0; j < kChunk / 64; j++) {
        const int pos = chunk * kChunk + j * 64 + lane;
        int p8 = 0;
        if (pos < len) {
            const float p = exp_f(scores[(size_t)qh * ld + pos] - mx) * cd;
            p8 = (int)roundf(p / as);
            p8 = p8 > 255 ? 255 : p8;
            if (p8_out) p8_out[(size_t)qh * len + pos] = (uint8_t)p8;
        }
        pb[j * 64 + lane] = (uint8_t)(p8 ^ 0x80);   // p8-128 as a signed byte
    }
    __syncthreads();
    // lane = output channel d; V block rows are [d][64 positions] = 64 contiguous bytes
    int acc = 0, vsum = 0;
#pragma unroll
    for (int j = 0; j < kChunk / 64; j++) {
        const int pos_blk = chunk * kChunk + j * 64;
        if (pos_blk < len) {
            const i32x4* vr = reinterpret_cast<const i32x4*>(vc + v_index(kvh, pos_blk, lane, max_pos));
            const i32x4* pr = reinterpret_cast<const i32x4*>(p_lds[g] + j * 16);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const i32x4 v = vr[c], p = pr[c];
                acc = __builtin_amdgcn_sdot4(p.x, v.x, acc, false); vsum = __builtin_amdgcn_sdot4(0x01010101, v.x, vsum, false);
                acc = __builtin_amdgcn_sdot4(p.y, v.y, acc, false); vsum = __builtin_amdgcn_sdot4(0x01010101, v.y, vsum, false);
                acc = __builtin_amdgcn_sdot4(p.z, v.z, acc, false); vsum = __builtin_amdgcn_sdot4(0x01010101, v.z, vsum, false);
                acc = __builtin_amdgcn_sdot4(p.w, v.w, acc, false); vsum = __builtin_amdgcn_sdot4(0x01010101, v.w, vsum, false);
            }
        }
    }
    atomicAdd(&o_acc[qh * kHd + lane], acc + 128 * vsum);
}

// ---- phase C ------------------------------------------------------------------------------
static __global__ __launch_bounds__(256) void dec_out_kernel(const int32_t* __restrict__ o_acc, const float* __restrict__ a_s,
                                                      const float* __restrict__ v_s, float* __restrict__ o, int n,
                                                      int group) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const int qh = i / kHd;
        o[i] = (float)o_acc[i] * a_s[qh] * v_s[qh / group];
    }
}

// ---- library-owned scratch for the stand-alone entry point -----------------------------------
struct DecodeScratch {
    float* scores = nullptr;   // [q_heads][len]
    float2* stats = nullptr;   // [q_heads][kMaxChunks]
    int32_t* o_acc = nullptr;  // [q_heads][64]
};

// The calling stream's scratch (stream_scratch), carved into the three arrays.
static int decode_scratch_of_stream(hipStream_t st, int q_heads, int len, DecodeScratch* out) {
    const size_t heads = q_heads > 32 ? q_heads : 32;
    const size_t need = (size_t)q_heads * len;
    const size_t elems = need > heads * 4096 ? need : heads * 4096;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t b_scores = up(elems * sizeof(float)), b_stats = up(heads * kMaxChunks * sizeof(float2)), b_acc = up(heads * kHd * sizeof(int32_t));
    void* base = nullptr;
    int rc = stream_scratch(kScratchMhaDecode, st, b_scores + b_stats + b_acc, &base);
    if (rc) return rc;
    char* p = static_cast<char*>(base);
    out->scores = reinterpret_cast<float*>(p);
    out->stats = reinterpret_cast<float2*>(p + b_scores);
    out->o_acc = reinterpret_cast<int32_t*>(p + b_scores + b_stats);
    return FLEXLLM_OK;
}

inline int mha_decode_launch(const int8_t* q8, const int8_t* kc, const int8_t* vc, const float* q_s, const float* k_s,
                      const float* v_s, const float* a_s, float* o, uint8_t* p8_out, float* scores, float2* stats,
                      int32_t* o_acc, int len, int q_heads, int kv_heads, int max_pos, hipStream_t st) {
    const int group = q_heads / kv_heads;
    const int nchunks = (len + kChunk - 1) / kChunk;
    dim3 grid(nchunks, kv_heads);
    dec_scores_kernel<<<grid, 64 * group, 0, st>>>(q8, kc, q_s, k_s, scores, stats, o_acc, nullptr, len, len, group, max_pos);
    dec_pv_kernel<<<grid, 64 * group, 0, st>>>(scores, stats, vc, a_s, o_acc, p8_out, nullptr, len, len, group, max_pos);
    const int n = q_heads * kHd;
    dec_out_kernel<<<(n + 255) / 256, 256, 0, st>>>(o_acc, a_s, v_s, o, n, group);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx

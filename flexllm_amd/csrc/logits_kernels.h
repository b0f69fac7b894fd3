// Greedy head: fp16 embedding lookup, tied fp16 lm_head GEMV (fp32 accumulate), argmax.
#pragma once
#include "common.h"
#include <hip/hip_fp16.h>

namespace fx {

using h16x8 = _Float16 __attribute__((ext_vector_type(8)));

// vocab > 0: a token id outside [0, vocab) is replaced by 0 and reported through *err = 2 (never looked up).
static __global__ __launch_bounds__(256) void embed_kernel(const __half* __restrict__ table, const int* __restrict__ token,
                                                    float* __restrict__ y, int hidden, int vocab = 0, int* __restrict__ err = nullptr) {
    int tk = token[0];
    if (vocab > 0 && (unsigned)tk >= (unsigned)vocab) {
        if (err && blockIdx.x == 0 && threadIdx.x == 0) err[0] = 2;
        tk = 0;
    }
    const size_t base = (size_t)tk * hidden;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < hidden; i += gridDim.x * 256) y[i] = __half2float(table[base + i]);
}

// Embeddings of a prompt: out[r] = fp32(E[tokens[r]]) for r < n, zero rows for n <= r < rows (padding to the prefill
// tile).  Ids outside [0, vocab) are replaced by 0 and reported through *err = 2.  One workgroup per row.
static __global__ __launch_bounds__(256) void embed_rows_kernel(const __half* __restrict__ table, const int* __restrict__ tokens,
                                                         int n, float* __restrict__ out, int hidden, int vocab, int* __restrict__ err) {
    const int r = blockIdx.x;
    float* dst = out + (size_t)r * hidden;
    if (r >= n) {
        for (int i = threadIdx.x; i < hidden; i += 256) dst[i] = 0.0f;
        return;
    }
    int tk = tokens[r];
    if ((unsigned)tk >= (unsigned)vocab) {
        if (err && threadIdx.x == 0) err[0] = 2;
        tk = 0;
    }
    const __half* src = table + (size_t)tk * hidden;
    for (int i = threadIdx.x; i < hidden; i += 256) dst[i] = __half2float(src[i]);
}

static __global__ void copy_int_kernel(const int* __restrict__ src, int* __restrict__ dst) { dst[0] = src[0]; }

// One wave per run of rows; lane reads 16-byte chunks (8 halves) lane, lane+64, ... of the row.
template <int NCH>
__global__ __launch_bounds__(256) void lm_head_kernel(const __half* __restrict__ table, const float* __restrict__ n,
                                                      float* __restrict__ logits, int vocab, int hidden, int rows_per_wave) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = gw * rows_per_wave;
    if (row0 >= vocab) return;
    const int nrows = min(rows_per_wave, vocab - row0);
    const int nchunks = hidden >> 3;
    float nv[NCH][8];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = lane + 64 * i;
#pragma unroll
        for (int e = 0; e < 8; e++) nv[i][e] = c < nchunks ? n[c * 8 + e] : 0.0f;
    }
    for (int r = 0; r < nrows; r++) {
        const h16x8* wr = reinterpret_cast<const h16x8*>(table + (size_t)(row0 + r) * hidden);
        h16x8 wv[NCH];
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = lane + 64 * i;
            wv[i] = c < nchunks ? __builtin_nontemporal_load(wr + c) : h16x8{0, 0, 0, 0, 0, 0, 0, 0};
        }
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < NCH; i++)
#pragma unroll
            for (int e = 0; e < 8; e++) acc += (float)wv[i][e] * nv[i][e];
        acc = wave_sum(acc);
        if (lane == 0) logits[row0 + r] = acc;
    }
}

// two-stage argmax, lowest index wins ties
static __global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ x, int n, float* __restrict__ pv,
                                                             int* __restrict__ pi) {
    __shared__ float sv[4];
    __shared__ int si[4];
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
        const float v = x[i];
        if (v > best || (v == best && i < bi)) { best = v; bi = i; }
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        const float ov = __shfl_xor(best, m);
        const int oi = __shfl_xor(bi, m);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++)
            if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
        pv[blockIdx.x] = best;
        pi[blockIdx.x] = bi;
    }
}
static __global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi,
                                                          int nparts, int* __restrict__ result) {
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
    if (threadIdx.x == 0) result[0] = bi == 0x7fffffff ? 0 : bi;
}

// ---- top-k sampling (Modules/Logits.h:145-279) ------------------------------------------------------------
// Each thread keeps the k best (value, index) of its share, ordered by value descending then index ascending; k
// rounds of a block-wide arg-max over the threads' current heads pop the top-k in that order.  Long rows go through
// two stages (128 workgroups over contiguous shares of the row, then one workgroup over their candidates: 23 us
// for 128256 logits where a single workgroup needs 230 us), short rows through the last stage alone.
// Thread 0 then does what the reference does with the k candidates: softmax with
// two partial sums (exp(v_k - v_0)), cumulative distribution, first k with rand < cdf[k] (else the last one).
// The reference orders EQUAL logits by its lane scan order instead of by index; the candidates' values, hence the
// probabilities, are the same either way, only which of two equal logits is reported can differ.
constexpr int kTopKMax = 16;
constexpr int kTopKThreads = 1024;
struct TopKOut { int* token; int* top_idx; float* top_val; float* top_prob; int* token_io; int* tokens_out; int* state; };

__device__ __forceinline__ bool topk_better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

// (value, index) as one 64-bit key whose unsigned order is "larger value first, then smaller index": the value's bits
// mapped monotonically to unsigned (sign bit flipped for positives, all bits for negatives; -0 is canonicalised to +0
// so that it ties with +0 as the float comparison does), the index complemented.
__device__ __forceinline__ unsigned long long topk_key(float v, int i) {
    const unsigned b = (unsigned)__float_as_int(v + 0.0f);
    const unsigned ord = b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
    return ((unsigned long long)ord << 32) | (unsigned)~i;
}
__device__ __forceinline__ float topk_key_value(unsigned long long k) {
    const unsigned ord = (unsigned)(k >> 32);
    return __int_as_float((int)(ord ^ ((ord >> 31) ? 0x80000000u : 0xFFFFFFFFu)));
}
__device__ __forceinline__ int topk_key_index(unsigned long long k) { return (int)~(unsigned)k; }
template <int MASK>
__device__ __forceinline__ unsigned long long topk_key_max_xor(unsigned long long k) {
    const unsigned lo = (unsigned)lane_xor_i<MASK>((int)(unsigned)k), hi = (unsigned)lane_xor_i<MASK>((int)(unsigned)(k >> 32));
    const unsigned long long o = ((unsigned long long)hi << 32) | lo;
    return o > k ? o : k;
}
__device__ __forceinline__ unsigned long long topk_key_wave_max(unsigned long long k) {
    k = topk_key_max_xor<1>(k); k = topk_key_max_xor<2>(k); k = topk_key_max_xor<4>(k);
    k = topk_key_max_xor<8>(k); k = topk_key_max_xor<16>(k); k = topk_key_max_xor<32>(k);
    return k;
}

// Block-wide selection: every thread holds a list sorted by (value descending, index ascending); top_k rounds of an
// arg-max over the threads' current heads pop the block's top_k in that order into f_val / f_idx (shared memory).
// Indices are distinct, so the winner's key identifies its owner: the thread whose head equals it advances.  (When
// fewer than top_k real entries exist the winner is the sentinel, which every exhausted list shows; advancing those
// changes nothing.)
template <int THREADS>
__device__ __forceinline__ void topk_block_select(const float (&val)[kTopKMax], const int (&idx)[kTopKMax], int top_k,
                                                  float* f_val, int* f_idx) {
    constexpr int NW = THREADS / 64;
    static_assert((NW & (NW - 1)) == 0 && NW <= 64, "waves per workgroup: a power of two");
    // wave winners of a round, double-buffered by round parity: a buffer is rewritten two rounds later, after the
    // barrier of the round in between, which no thread passes before it has read this round's entries
    __shared__ unsigned long long s_key[2][NW];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    int head = 0;                                   // this thread's best not yet taken
    for (int r = 0; r < top_k; r++) {
        float bv = -1e32f; int bi = 0x7fffffff;
#pragma unroll
        for (int k = 0; k < kTopKMax; k++) if (k == head) { bv = val[k]; bi = idx[k]; }
        if (head >= top_k) { bv = -1e32f; bi = 0x7fffffff; }
        const unsigned long long mine = topk_key(bv, bi);
        const unsigned long long wmax = topk_key_wave_max(mine);
        if (lane == 0) s_key[r & 1][wave] = wmax;
        __syncthreads();
        // every wave reduces the NW wave winners itself (each group of NW lanes holds all of them), so every thread
        // learns the round's winner without a second exchange
        unsigned long long win = s_key[r & 1][lane & (NW - 1)];
        if constexpr (NW > 1) win = topk_key_max_xor<1>(win);
        if constexpr (NW > 2) win = topk_key_max_xor<2>(win);
        if constexpr (NW > 4) win = topk_key_max_xor<4>(win);
        if constexpr (NW > 8) win = topk_key_max_xor<8>(win);
        if constexpr (NW > 16) win = topk_key_max_xor<16>(win);
        if constexpr (NW > 32) win = topk_key_max_xor<32>(win);
        if (t == 0) { f_val[r] = topk_key_value(win); f_idx[r] = topk_key_index(win); }
        if (mine == win) head++;
    }
    __syncthreads();
}

// Sorted insertion of one candidate (k is small; statically indexed so that the lists stay in registers).
__device__ __forceinline__ void topk_insert(float (&val)[kTopKMax], int (&idx)[kTopKMax], int top_k, float cv, int ci) {
#pragma unroll
    for (int k = 0; k < kTopKMax; k++) {
        if (k < top_k && topk_better(cv, ci, val[k], idx[k])) {
            const float tv = val[k]; const int ti = idx[k];
            val[k] = cv; idx[k] = ci; cv = tv; ci = ti;
        }
    }
}

// What the reference does with the k candidates (values in rank order): softmax with two partial sums of
// exp(v_k - v_0), cumulative distribution, the first k with rnd < cdf[k] (else the last one).  Returns the rank of the
// sampled candidate; prob receives the probabilities.  Loops run over the compile-time maximum with a predicate so
// that the small arrays stay in registers.  One thread calls this.
__device__ __forceinline__ int topk_sample_rank(const float* f_val, int top_k, float rnd, int enable_sub_max, float (&prob)[kTopKMax]) {
    float cdf[kTopKMax];
    float sum_partial[2] = {0.0f, 0.0f};
    const float v0 = f_val[0];
#pragma unroll
    for (int k = 0; k < kTopKMax; k++) {
        prob[k] = 0.0f;
        if (k < top_k) {
            const float e = enable_sub_max ? expf(f_val[k] - v0) : expf(f_val[k]);
            prob[k] = e;
            sum_partial[k % 2] += e;
        }
    }
    const float sum = sum_partial[0] + sum_partial[1];
#pragma unroll
    for (int k = 0; k < kTopKMax; k++) if (k < top_k) prob[k] = prob[k] / sum;
    cdf[0] = prob[0];
#pragma unroll
    for (int k = 1; k < kTopKMax; k++) cdf[k] = k < top_k ? prob[k] + cdf[k - 1] : cdf[k - 1];
    int selected = top_k - 1;
#pragma unroll
    for (int k = kTopKMax - 1; k >= 0; k--)
        if (k < top_k && rnd < cdf[k]) selected = k;                    // ends on the first k with rnd < cdf[k]
    return selected;
}

// First stage for long rows: workgroup g selects the top_k of its contiguous share of the logits and writes them,
// in order, to cand_val / cand_idx [g * top_k ...]; unused places carry the sentinel (-1e32, 0x7fffffff).  The global
// top_k is a subset of the union, and the second stage (topk_sample_kernel with in_idx) orders it the same way.
constexpr int kTopKParts = 128;
constexpr int kTopKPartThreads = 256;
static __global__ __launch_bounds__(kTopKPartThreads) void topk_partial_kernel(const float* __restrict__ logits, int n, int top_k,
                                                                              float* __restrict__ cand_val, int* __restrict__ cand_idx) {
    __shared__ float f_val[kTopKMax];
    __shared__ int f_idx[kTopKMax];
    const int chunk = (n + gridDim.x - 1) / gridDim.x;
    const int begin = blockIdx.x * chunk, end = min(n, begin + chunk);
    float val[kTopKMax];
    int idx[kTopKMax];
#pragma unroll
    for (int k = 0; k < kTopKMax; k++) { val[k] = -1e32f; idx[k] = 0x7fffffff; }
    // four loads in flight per thread (a share of the 128256-entry vocabulary is 1002 logits: one batch)
    for (int i0 = begin + threadIdx.x; i0 < end; i0 += 4 * kTopKPartThreads) {
        float lv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) lv[u] = i0 + u * kTopKPartThreads < end ? logits[i0 + u * kTopKPartThreads] : 0.0f;
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (i0 + u * kTopKPartThreads < end) topk_insert(val, idx, top_k, lv[u], i0 + u * kTopKPartThreads);
    }
    topk_block_select<kTopKPartThreads>(val, idx, top_k, f_val, f_idx);
    if (threadIdx.x < top_k) {
        cand_val[blockIdx.x * top_k + threadIdx.x] = f_val[threadIdx.x];
        cand_idx[blockIdx.x * top_k + threadIdx.x] = f_idx[threadIdx.x];
    }
}

// in_idx == NULL: logits[i] is the logit of token i.  Otherwise (second stage) logits / in_idx are n candidates.
// THREADS: 1024 for a whole short row, 256 for the few hundred candidates of the second stage (the selection rounds
// cost issue slots per wave, and all waves of the one workgroup share a CU).
template <int THREADS>
static __global__ __launch_bounds__(THREADS) void topk_sample_kernel(const float* __restrict__ logits, const int* __restrict__ in_idx,
                                                                    int n, int top_k, const float* __restrict__ rand_ptr,
                                                                    int rand_index_from_state, int enable_sub_max, TopKOut out) {
    __shared__ float f_val[kTopKMax];
    __shared__ int f_idx[kTopKMax];
    const int t = threadIdx.x;
    float val[kTopKMax];
    int idx[kTopKMax];
#pragma unroll
    for (int k = 0; k < kTopKMax; k++) { val[k] = -1e32f; idx[k] = 0x7fffffff; }
    for (int i = t; i < n; i += THREADS) topk_insert(val, idx, top_k, logits[i], in_idx ? in_idx[i] : i);
    topk_block_select<THREADS>(val, idx, top_k, f_val, f_idx);
    if (t < top_k && f_idx[t] == 0x7fffffff) f_idx[t] = -1;
    __syncthreads();
    if (t == 0) {
        float prob[kTopKMax];
        const float rnd = rand_ptr[rand_index_from_state && out.state ? out.state[1] : 0];
        const int selected = topk_sample_rank(f_val, top_k, rnd, enable_sub_max, prob);
        const int tok = f_idx[selected];
        if (out.token) out.token[0] = tok;
#pragma unroll
        for (int k = 0; k < kTopKMax; k++) {
            if (k < top_k) {
                if (out.top_idx) out.top_idx[k] = f_idx[k];
                if (out.top_val) out.top_val[k] = f_val[k];
                if (out.top_prob) out.top_prob[k] = prob[k];
            }
        }
        if (out.state) {                            // generation loop: hand the token over and advance position / step
            out.token_io[0] = tok;
            out.tokens_out[out.state[1]] = tok;
            out.state[0] += 1;
            out.state[1] += 1;
        }
    }
}

constexpr int kArgmaxParts = 256;
// (the stand-alone arg-max and sampling entry points keep their candidate buffers in the calling stream's scratch,
// a model object owns buffers of its own)

inline int argmax_launch(const float* x, int n, int* result, float* pv, int* pi, hipStream_t st) {
    argmax_partial_kernel<<<kArgmaxParts, 256, 0, st>>>(x, n, pv, pi);
    argmax_final_kernel<<<1, 64, 0, st>>>(pv, pi, kArgmaxParts, result);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

inline int lm_head_launch(const uint16_t* embed, const float* n, float* logits, int vocab, int hidden, hipStream_t st) {
    const int nch = (hidden / 8 + 63) / 64;
    const int rpw = 16;
    const int waves = (vocab + rpw - 1) / rpw;
    const int grid = (waves + 3) / 4;
    const __half* t = reinterpret_cast<const __half*>(embed);
    if (nch <= 1) lm_head_kernel<1><<<grid, 256, 0, st>>>(t, n, logits, vocab, hidden, rpw);
    else if (nch <= 2) lm_head_kernel<2><<<grid, 256, 0, st>>>(t, n, logits, vocab, hidden, rpw);
    else if (nch <= 4) lm_head_kernel<4><<<grid, 256, 0, st>>>(t, n, logits, vocab, hidden, rpw);
    else lm_head_kernel<8><<<grid, 256, 0, st>>>(t, n, logits, vocab, hidden, rpw);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx

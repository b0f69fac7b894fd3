// Causal int8 prefill attention (GQA) on MFMA, reading K and V from the layer's int8 cache.
//
// A workgroup owns 32 consecutive queries of one head; its waves split the key tiles (32 keys) up to the
// diagonal.
// The score tile is computed TRANSPOSED, S^T = K_tile . Q_tile^T, so that in the 32x32 accumulator layout a
// lane holds 16 scores of ONE query (column l%32; keys 8a+4g+b for register 4a+b, g = l/32).  That is also
// the A-operand shape of the second matrix product P.V (row = query l%32, 16 k-values for k-group g), so the
// quantised probabilities never leave the registers; V's B operand is gathered in the same key order from
// the cache's transposed 64-position blocks ([channel][position]: four 4-byte runs per lane).
//
// The reference normalises by the full-row sum BEFORE rounding the probabilities to uint8, so the wave makes
// two passes over its key tiles: pass 1 keeps a running max / running sum of exponentials per query, pass 2
// recomputes the scores (64-deep dot products: cheap), forms p = exp(s-max)*(1/sum), P = min(255,
// round(p/A_s)) and accumulates P.V.  P is unsigned and the MFMA is signed x signed: (P-128).V is
// accumulated and 128*colsum(V) over the same keys is added at the end, both exact in int32.
#pragma once
#include "attn_decode_kernels.h"

namespace fx {

constexpr int kPfTile = 32;

__device__ __forceinline__ i32x16 zero16() {
    i32x16 z;
#pragma unroll
    for (int r = 0; r < 16; r++) z[r] = 0;
    return z;
}

// grid (s/32 * q_heads), 64 * kPfWaves threads: the waves of a workgroup share one block of 32 queries and split
// its key tiles round-robin (tile kt goes to wave kt % kPfWaves).  Row statistics are merged through LDS after pass 1;
// the int32 P.V partial accumulators of the waves are added in LDS after pass 2 (integer adds: exact).
//
// Work per query block grows linearly with its index (causal), and workgroups b, b+P, b+2P, ... (P = number of
// CUs) end up resident on the same CU.  The (block, head) items are therefore taken in order of decreasing
// length and dealt out in snake order (first deal forwards, second backwards, ...): every CU gets the same total.
constexpr int kPfWaves = 4;        // waves per workgroup (8 measured slower: the kernel is bound by VALU throughput, not by the longest block)
static __global__ __launch_bounds__(64 * kPfWaves) void pf_attention_kernel(const int8_t* __restrict__ q8, const int8_t* __restrict__ kc,
                                                                  const int8_t* __restrict__ vc, const float* __restrict__ q_s,
                                                                  const float* __restrict__ k_s, const float* __restrict__ v_s,
                                                                  const float* __restrict__ a_s, float* __restrict__ o,
                                                                  uint8_t* __restrict__ p8_out, int s, int q_heads, int group,
                                                                  int max_pos, int period) {
    __shared__ float lds_m[kPfWaves][32], lds_l[kPfWaves][32];
    __shared__ int lds_acc[64][35];            // [lane][16 acc0 | 16 acc1 | vsum0 | vsum1], odd pitch against bank conflicts
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n_items = (int)gridDim.x, nqb = s / kPfTile;
    const int round = (int)blockIdx.x / period, c = (int)blockIdx.x % period;
    const int in_round = min(period, n_items - round * period);
    const int item = round * period + ((round & 1) ? in_round - 1 - c : c);   // index into the items sorted by decreasing length
    const int qb = nqb - 1 - item / q_heads;
    const int q0 = qb * kPfTile;
    const int h = item % q_heads, kvh = h / group;
    const int col = lane & 31, g = lane >> 5;
    const int query = q0 + col;
    const float sq = q_s[h], sk = k_s[kvh], as = 1.0f * a_s[h];

    // B operand of S^T = K.Q^T: this lane's query row, 16 d-bytes of k-group g, two k-steps (d 0..31, 32..63)
    const int8_t* qrow = q8 + ((size_t)query * q_heads + h) * kHd;
    const i32x4 qf0 = *reinterpret_cast<const i32x4*>(qrow + g * 16);
    const i32x4 qf1 = *reinterpret_cast<const i32x4*>(qrow + 32 + g * 16);

    auto load_k = [&](int k0, i32x4& kf0, i32x4& kf1) {
        const int8_t* krow = kc + k_index(kvh, k0 + col, max_pos);
        kf0 = *reinterpret_cast<const i32x4*>(krow + g * 16);
        kf1 = *reinterpret_cast<const i32x4*>(krow + 32 + g * 16);
    };
    auto score_tile = [&](int k0, const i32x4& kf0, const i32x4& kf1, float (&sc)[16]) {
        i32x16 acc = zero16();
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf0, qf0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf1, qf1, acc, 0, 0, 0);
        if (k0 == q0) {                                   // only the diagonal tile has keys beyond the query (uniform branch)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = k0 + (r >> 2) * 8 + g * 4 + (r & 3);
                const float v = (float)acc[r] * sq * sk;
                sc[r] = key <= query ? v : -1e32f;
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) sc[r] = (float)acc[r] * sq * sk;
        }
    };

    const int ntiles = qb + 1;
    for (int i = threadIdx.x; i < 64 * 35; i += 64 * kPfWaves) (&lds_acc[0][0])[i] = 0;
    // ---- pass 1: row max and row sum of exponentials over this wave's tiles ----
    float m_run = -1e32f, l_run = 0.0f;
    {
        i32x4 kf0, kf1, nf0, nf1;
        if (wave < ntiles) load_k(wave * kPfTile, kf0, kf1);
        for (int kt = wave; kt < ntiles; kt += kPfWaves) {
            if (kt + kPfWaves < ntiles) load_k((kt + kPfWaves) * kPfTile, nf0, nf1);
            float sc[16];
            score_tile(kt * kPfTile, kf0, kf1, sc);
            float mt = sc[0];
#pragma unroll
            for (int r = 1; r < 16; r++) mt = fmaxf(mt, sc[r]);
            const float m_new = fmaxf(m_run, mt);
            float sum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) sum += exp_f<false>(sc[r] - m_new);
            l_run = l_run * exp_f<false>(m_run - m_new) + sum;
            m_run = m_new;
            kf0 = nf0; kf1 = nf1;
        }
    }
    {   // merge the two lanes that share a query, then the waves
        const float m_o = lane_xor_f<32>(m_run), l_o = lane_xor_f<32>(l_run);
        const float mw = fmaxf(m_run, m_o);
        const float lw = l_run * exp_f(m_run - mw) + l_o * exp_f(m_o - mw);
        if (g == 0) { lds_m[wave][col] = mw; lds_l[wave][col] = lw; }
    }
    __syncthreads();
    float mx = lds_m[0][col];
#pragma unroll
    for (int w = 1; w < kPfWaves; w++) mx = fmaxf(mx, lds_m[w][col]);
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kPfWaves; w++) total += lds_l[w][col] * exp_f(lds_m[w][col] - mx);
    const float cd = 1.0f / total;
    const bool fast_q = quant_fast_ok(as);
    const float ras = 1.0f / as;

    // ---- pass 2: probabilities, partial P.V over this wave's tiles ----
    i32x16 oacc0 = zero16(), oacc1 = zero16();
    int vsum0 = 0, vsum1 = 0;
    {
        i32x4 kf0, kf1, nf0, nf1;
        if (wave < ntiles) load_k(wave * kPfTile, kf0, kf1);
        for (int kt = wave; kt < ntiles; kt += kPfWaves) {
            const int k0 = kt * kPfTile;
            if (kt + kPfWaves < ntiles) load_k((kt + kPfWaves) * kPfTile, nf0, nf1);
            // B operand of P.V: V[key][d] for this lane's channel d = col (+32) and the lane's 16 keys, gathered
            // from the cache's [d][64 pos] blocks; issued before the exponentials so that it is in flight
            const int8_t* vblk = vc + v_index(kvh, k0, 0, max_pos);
            i32x4 vf0, vf1;
#pragma unroll
            for (int a = 0; a < 4; a++) {
                vf0[a] = *reinterpret_cast<const int*>(vblk + (size_t)col * kVBlock + a * 8 + g * 4);
                vf1[a] = *reinterpret_cast<const int*>(vblk + (size_t)(col + 32) * kVBlock + a * 8 + g * 4);
            }
            float sc[16];
            score_tile(k0, kf0, kf1, sc);
            i32x4 pf;
#pragma unroll
            for (int a = 0; a < 4; a++) {
                // four probabilities -> four bytes; round(pr / as) through the reciprocal, redone with the division
                // for the whole group when one of them comes near a rounding tie
                float pr[4];
                int p8[4];
                bool redo = !fast_q;
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    pr[b] = exp_f<false>(sc[a * 4 + b] - mx) * cd;
                    const float qv = pr[b] * ras;               // >= 0: round half up = truncate(qv + 0.5)
                    redo |= fabsf(__builtin_amdgcn_fractf(qv) - 0.5f) < 1e-4f;
                    p8[b] = (int)(qv + 0.5f);
                }
                if (redo) {
#pragma unroll
                    for (int b = 0; b < 4; b++) p8[b] = (int)roundf(pr[b] / as);
                }
                uint32_t packed = 0;
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const int pq = p8[b] > 255 ? 255 : p8[b];
                    if (p8_out) {
                        const int key = k0 + a * 8 + g * 4 + b;
                        p8_out[((size_t)h * s + query) * s + key] = (uint8_t)pq;
                    }
                    packed |= (uint32_t)((pq ^ 0x80) & 0xff) << (8 * b);
                }
                pf[a] = (int)packed;
            }
#pragma unroll
            for (int a = 0; a < 4; a++) {
                vsum0 = __builtin_amdgcn_sdot4(0x01010101, vf0[a], vsum0, false);
                vsum1 = __builtin_amdgcn_sdot4(0x01010101, vf1[a], vsum1, false);
            }
            oacc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(pf, vf0, oacc0, 0, 0, 0);
            oacc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(pf, vf1, oacc1, 0, 0, 0);
            kf0 = nf0; kf1 = nf1;
        }
    }
    // add the waves' partial accumulators (lds_acc was zeroed before pass 1; two barriers have passed)
    if (wave < ntiles) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            atomicAdd(&lds_acc[lane][r], oacc0[r]);
            atomicAdd(&lds_acc[lane][16 + r], oacc1[r]);
        }
        atomicAdd(&lds_acc[lane][32], vsum0);
        atomicAdd(&lds_acc[lane][33], vsum1);
    }
    __syncthreads();
    const int vs0 = lds_acc[lane][32] + lds_acc[lane ^ 32][32];
    const int vs1 = lds_acc[lane][33] + lds_acc[lane ^ 32][33];
    const float sv = v_s[kvh], sa = a_s[h];
#pragma unroll
    for (int rr = 0; rr < 16 / kPfWaves; rr++) {              // each wave writes its share of the 16 accumulator registers
        const int r = wave * (16 / kPfWaves) + rr;
        const int row = q0 + (r >> 2) * 8 + g * 4 + (r & 3);
        float* orow = o + ((size_t)row * q_heads + h) * kHd;
        orow[col] = (float)(lds_acc[lane][r] + 128 * vs0) * sa * sv;
        orow[col + 32] = (float)(lds_acc[lane][16 + r] + 128 * vs1) * sa * sv;
    }
}

// The same attention for rows of at most kPfWaves * kPfCachedTiles * 32 = 1024 keys, with every score tile of the
// wave held in registers (8 tiles x 16 values per lane): the scores are computed ONCE as integers, the row maximum is
// an integer maximum (the dequantisation is monotonic), the exponentials are computed ONCE with the final maximum and
// replace the integers in place, and the second pass only scales, rounds and multiplies with V.  This is also the
// reference's own order (maximum, then exponentials and their sum, then probabilities from the same exponentials).
// Per probability: one exponential instead of two, one dequantisation instead of two, K read once.
constexpr int kPfCachedTiles = 8;
static __global__ __launch_bounds__(64 * kPfWaves, 2) void pf_attention_cached_kernel(
    const int8_t* __restrict__ q8, const int8_t* __restrict__ kc, const int8_t* __restrict__ vc, const float* __restrict__ q_s,
    const float* __restrict__ k_s, const float* __restrict__ v_s, const float* __restrict__ a_s, float* __restrict__ o,
    uint8_t* __restrict__ p8_out, int s, int q_heads, int group, int max_pos, int period) {
    __shared__ int lds_mi[kPfWaves][32];
    __shared__ float lds_l[kPfWaves][32];
    __shared__ int lds_acc[64][35];            // [lane][16 acc0 | 16 acc1 | vsum0 | vsum1], odd pitch against bank conflicts
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n_items = (int)gridDim.x, nqb = s / kPfTile;
    const int round = (int)blockIdx.x / period, c = (int)blockIdx.x % period;
    const int in_round = min(period, n_items - round * period);
    const int item = round * period + ((round & 1) ? in_round - 1 - c : c);   // index into the items sorted by decreasing length
    const int qb = nqb - 1 - item / q_heads;
    const int q0 = qb * kPfTile;
    const int h = item % q_heads, kvh = h / group;
    const int col = lane & 31, g = lane >> 5;
    const int query = q0 + col;
    const float sq = q_s[h], sk = k_s[kvh], as = 1.0f * a_s[h];

    const int8_t* qrow = q8 + ((size_t)query * q_heads + h) * kHd;
    const i32x4 qf0 = *reinterpret_cast<const i32x4*>(qrow + g * 16);
    const i32x4 qf1 = *reinterpret_cast<const i32x4*>(qrow + 32 + g * 16);
    auto load_k = [&](int k0, i32x4& kf0, i32x4& kf1) {
        const int8_t* krow = kc + k_index(kvh, k0 + col, max_pos);
        kf0 = *reinterpret_cast<const i32x4*>(krow + g * 16);
        kf1 = *reinterpret_cast<const i32x4*>(krow + 32 + g * 16);
    };
    const int ntiles = qb + 1;                                 // <= kPfWaves * kPfCachedTiles (checked by the launcher)
    for (int i = threadIdx.x; i < 64 * 35; i += 64 * kPfWaves) (&lds_acc[0][0])[i] = 0;

    // ---- pass 0: integer scores of this wave's tiles (kept), integer row maximum ----
    constexpr int kMasked = -0x7fffffff - 1;
    int tv[kPfCachedTiles][16];
    int imax = kMasked;
    {
        i32x4 kf0, kf1, nf0, nf1;
        if (wave < ntiles) load_k(wave * kPfTile, kf0, kf1);
#pragma unroll
        for (int i = 0; i < kPfCachedTiles; i++) {
            const int kt = wave + kPfWaves * i;
            if (kt < ntiles) {
                if (kt + kPfWaves < ntiles) load_k((kt + kPfWaves) * kPfTile, nf0, nf1);
                i32x16 acc = zero16();
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf0, qf0, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf1, qf1, acc, 0, 0, 0);
                if (kt == qb) {                                // only the diagonal tile has keys beyond the query
#pragma unroll
                    for (int r = 0; r < 16; r++) tv[i][r] = (q0 + (r >> 2) * 8 + g * 4 + (r & 3)) <= query ? acc[r] : kMasked;
                } else {
#pragma unroll
                    for (int r = 0; r < 16; r++) tv[i][r] = acc[r];
                }
#pragma unroll
                for (int r = 0; r < 16; r++) imax = max(imax, tv[i][r]);
                kf0 = nf0; kf1 = nf1;
            }
        }
    }
    imax = max(imax, lane_xor_i<32>(imax));                    // the two lanes that share a query
    if (g == 0) lds_mi[wave][col] = imax;                      // a wave without tiles contributes the masked value
    __syncthreads();
    int im = lds_mi[0][col];
#pragma unroll
    for (int w = 1; w < kPfWaves; w++) im = max(im, lds_mi[w][col]);
    const float mx = (float)im * sq * sk;                      // int -> float and the positive scales keep the order

    // ---- pass 1: exponentials with the final maximum, in place; row sum ----
    float lsum = 0.0f;
#pragma unroll
    for (int i = 0; i < kPfCachedTiles; i++) {
        const int kt = wave + kPfWaves * i;
        if (kt < ntiles) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float e = exp_f<false>((float)tv[i][r] * sq * sk - mx);
                if (kt == qb && tv[i][r] == kMasked) e = 0.0f;  // masked keys count as exp(-1e32 - max) = 0 whatever the scales
                tv[i][r] = __float_as_int(e);
                lsum += e;
            }
        }
    }
    lsum = lsum + lane_xor_f<32>(lsum);
    if (g == 0) lds_l[wave][col] = lsum;
    __syncthreads();
    float total = lds_l[0][col];
#pragma unroll
    for (int w = 1; w < kPfWaves; w++) total += lds_l[w][col];
    const float cd = 1.0f / total;
    const bool fast_q = quant_fast_ok(as);
    const float ras = 1.0f / as;

    // ---- pass 2: probabilities from the kept exponentials, partial P.V ----
    i32x16 oacc0 = zero16(), oacc1 = zero16();
    int vsum0 = 0, vsum1 = 0;
#pragma unroll
    for (int i = 0; i < kPfCachedTiles; i++) {
        const int kt = wave + kPfWaves * i;
        if (kt < ntiles) {
            const int k0 = kt * kPfTile;
            // B operand of P.V: V[key][d] for this lane's channels col, col+32 and its 16 keys, gathered from the
            // cache's [d][64 pos] blocks; issued before the rounding work so that it is in flight
            const int8_t* vblk = vc + v_index(kvh, k0, 0, max_pos);
            i32x4 vf0, vf1;
#pragma unroll
            for (int a = 0; a < 4; a++) {
                vf0[a] = *reinterpret_cast<const int*>(vblk + (size_t)col * kVBlock + a * 8 + g * 4);
                vf1[a] = *reinterpret_cast<const int*>(vblk + (size_t)(col + 32) * kVBlock + a * 8 + g * 4);
            }
            i32x4 pf;
#pragma unroll
            for (int a = 0; a < 4; a++) {
                float pr[4];
                int p8[4];
                bool redo = !fast_q;
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    pr[b] = __int_as_float(tv[i][a * 4 + b]) * cd;
                    const float qv = pr[b] * ras;               // >= 0: round half up = truncate(qv + 0.5)
                    redo |= fabsf(__builtin_amdgcn_fractf(qv) - 0.5f) < 1e-4f;
                    p8[b] = (int)(qv + 0.5f);
                }
                if (redo) {
#pragma unroll
                    for (int b = 0; b < 4; b++) p8[b] = (int)roundf(pr[b] / as);
                }
                uint32_t packed = 0;
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const int pq = p8[b] > 255 ? 255 : p8[b];
                    if (p8_out) {
                        const int key = k0 + a * 8 + g * 4 + b;
                        p8_out[((size_t)h * s + query) * s + key] = (uint8_t)pq;
                    }
                    packed |= (uint32_t)((pq ^ 0x80) & 0xff) << (8 * b);
                }
                pf[a] = (int)packed;
            }
#pragma unroll
            for (int a = 0; a < 4; a++) {
                vsum0 = __builtin_amdgcn_sdot4(0x01010101, vf0[a], vsum0, false);
                vsum1 = __builtin_amdgcn_sdot4(0x01010101, vf1[a], vsum1, false);
            }
            oacc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(pf, vf0, oacc0, 0, 0, 0);
            oacc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(pf, vf1, oacc1, 0, 0, 0);
        }
    }
    if (wave < ntiles) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            atomicAdd(&lds_acc[lane][r], oacc0[r]);
            atomicAdd(&lds_acc[lane][16 + r], oacc1[r]);
        }
        atomicAdd(&lds_acc[lane][32], vsum0);
        atomicAdd(&lds_acc[lane][33], vsum1);
    }
    __syncthreads();
    const int vs0 = lds_acc[lane][32] + lds_acc[lane ^ 32][32];
    const int vs1 = lds_acc[lane][33] + lds_acc[lane ^ 32][33];
    const float sv = v_s[kvh], sa = a_s[h];
#pragma unroll
    for (int rr = 0; rr < 16 / kPfWaves; rr++) {
        const int r = wave * (16 / kPfWaves) + rr;
        const int row = q0 + (r >> 2) * 8 + g * 4 + (r & 3);
        float* orow = o + ((size_t)row * q_heads + h) * kHd;
        orow[col] = (float)(lds_acc[lane][r] + 128 * vs0) * sa * sv;
        orow[col + 32] = (float)(lds_acc[lane][16 + r] + 128 * vs1) * sa * sv;
    }
}

inline int mha_prefill_launch(const int8_t* q8, const int8_t* kc, const int8_t* vc, const float* q_s, const float* k_s,
                              const float* v_s, const float* a_s, float* o, uint8_t* p8_out, int s, int q_heads,
                              int kv_heads, int max_pos, hipStream_t st) {
    static int n_cu = 0;
    if (!n_cu) {
        int dev = 0;
        FX_HIP(hipGetDevice(&dev));
        FX_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
        if (n_cu <= 0) n_cu = 256;
    }
    static const bool no_cached = getenv("FLEXLLM_ATTN_RECOMPUTE") != nullptr;      // forces the two-pass kernel (comparison runs)
    if (s <= kPfTile * kPfWaves * kPfCachedTiles && !no_cached)
        pf_attention_cached_kernel<<<(s / kPfTile) * q_heads, 64 * kPfWaves, 0, st>>>(q8, kc, vc, q_s, k_s, v_s, a_s, o, p8_out, s, q_heads,
                                                                          q_heads / kv_heads, max_pos, n_cu);
    else
        pf_attention_kernel<<<(s / kPfTile) * q_heads, 64 * kPfWaves, 0, st>>>(q8, kc, vc, q_s, k_s, v_s, a_s, o, p8_out, s, q_heads,
                                                                   q_heads / kv_heads, max_pos, n_cu);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx

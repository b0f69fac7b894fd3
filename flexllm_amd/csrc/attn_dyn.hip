// int8 GQA attention with DYNAMIC per-(token, head) scales, prefill and decode.
//
// Q, K and V come from the library's per-(token, head) symmetric quantiser (Modules/quant.h:527-617,
// flexllm_head_quant_sym_i8): one scale per token and head, so a score is dequantised per key,
//     a[i][j] = (float(q8_i . k8_j) * Q_s[i][h]) * K_s[j][kvh]          (Modules/quant.h:225-246),
// with Q_s = s_q / q_scale_div (sqrt(head_dim), the factor the static path folds into Q's scale).  V's per-token scale
// varies along the reduction of P.V, so it is folded into the probabilities before they are quantised:
//     p'[j] = softmax(a)[j] * V_s[j][kvh];   s_p = max_j p'[j] / 127 (0 -> 1);   P8 = round(p' / s_p)   (int8, 0..127)
//     o[d]  = float(sum_j P8[j] * v8[j][d]) * s_p  (* v_ch_s[kvh][d], the reference library's per-channel V scale).
// P is signed here (0..127), so the MFMA / dot products need no offset trick.
//
// Prefill: the tiling of attn_prefill.h (32 queries x one head per workgroup, eight waves split the key tiles,
// S^T = K.Q^T so that the probabilities land in the A-operand layout of P.V).  The row needs two global quantities
// before a probability can be rounded: the softmax denominator and the maximum of p'.  Rows of up to 1024 keys keep
// their scores in registers between those steps (pf_attention_dyn_cached_kernel); longer rows go over the wave's tiles in
// three passes and form the scores again in each (64-deep dot products on the matrix cores: cheap).
// Decode: the chunked kernels of attn_decode_kernels.h with one more kernel for the row maximum of p'.
#include "attn_prefill.h"
#include "gemv_i8.h"

namespace fx {

struct DynScales {
    const float *q_s, *k_s, *v_s, *v_ch_s;   // [rows][q_heads], [max_pos][kv_heads] x2, optional [kv_heads][64]
    float q_div;
};

// Rows of any length: three passes over the wave's tiles, the scores formed again in each.  The K rows are loaded in the
// permuted order of attn_prefill.h (a lane's 16 values are 16 consecutive keys); the tile's K and V scales are fetched by
// the wave's lanes (one key each), parked in a wave-private corner of LDS and read back as four 16-byte words per lane.
template <bool kStoreP>
static __global__ __launch_bounds__(64 * kPfWaves) void pf_attention_dyn_kernel(
    const int8_t* __restrict__ q8, const int8_t* __restrict__ kc, const int8_t* __restrict__ vc, DynScales sc,
    float* __restrict__ o, int8_t* __restrict__ p8_out, float* __restrict__ p_s_out, int s, int q_heads, int kv_heads,
    int max_pos, int period) {
    __shared__ float lds_m[kPfWaves][32], lds_l[kPfWaves][32], lds_pm[kPfWaves][32], lds_sp[32];
    __shared__ int lds_acc[64][33];            // [lane][16 acc0 | 16 acc1], odd pitch against bank conflicts
    __shared__ __attribute__((aligned(16))) float lds_sc[kPfWaves][2][kPfTile];   // per wave: K scales, V scales of the current tile
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int group = q_heads / kv_heads;
    const PfItem it = pf_item(s, q_heads, group, period);
    const int col = it.col, g = it.g, query = it.query, ntiles = it.ntiles, kvh = it.kvh, h = it.h;
    const float sq = sc.q_s[(size_t)query * q_heads + h] / sc.q_div;

    const int8_t* qrow = q8 + ((size_t)query * q_heads + h) * kHd;
    const i32x4 qf0 = *reinterpret_cast<const i32x4*>(qrow + g * 16);
    const i32x4 qf1 = *reinterpret_cast<const i32x4*>(qrow + 32 + g * 16);
    const int krow_in_tile = pf_key_of_row(col);
    const float* scale_tab = g == 0 ? sc.k_s : sc.v_s;        // lanes 0..31 fetch the K scales of the tile's keys, lanes 32..63 the V scales
    // scores of tile kt (register r = key k0 + 16 g + r, masked beyond the query) and, on request, the V scales of the same keys
    auto tile = [&](int kt, float (&scv)[16], float (&vs)[16], bool want_vs) {
        const int k0 = kt * kPfTile;
        const int8_t* krow = kc + k_index(kvh, k0 + krow_in_tile, max_pos);
        const i32x4 kf0 = *reinterpret_cast<const i32x4*>(krow + g * 16);
        const i32x4 kf1 = *reinterpret_cast<const i32x4*>(krow + 32 + g * 16);
        lds_sc[wave][g][col] = scale_tab[(size_t)(k0 + col) * kv_heads + kvh];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();                       // the corner is private to the wave: its LDS accesses complete in order
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        i32x16 acc = zero16();
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf0, qf0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf1, qf1, acc, 0, 0, 0);
#pragma unroll
        for (int a = 0; a < 4; a++) {
            const float4 ks4 = *reinterpret_cast<const float4*>(&lds_sc[wave][0][16 * g + 4 * a]);
            const float ks[4] = {ks4.x, ks4.y, ks4.z, ks4.w};
            if (want_vs) {
                const float4 vs4 = *reinterpret_cast<const float4*>(&lds_sc[wave][1][16 * g + 4 * a]);
                vs[4 * a] = vs4.x; vs[4 * a + 1] = vs4.y; vs[4 * a + 2] = vs4.z; vs[4 * a + 3] = vs4.w;
            }
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const float v = (float)acc[4 * a + b] * sq * ks[b];
                scv[4 * a + b] = (k0 + 16 * g + 4 * a + b <= query) ? v : -1e32f;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();                       // reads of this tile's scales before the next tile's writes
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    for (int i = threadIdx.x; i < 64 * 33; i += 64 * kPfWaves) (&lds_acc[0][0])[i] = 0;
    float scv[16], vs[16];
    // ---- pass 1: row maximum and sum of exponentials over this wave's tiles ----
    float m_run = -1e32f, l_run = 0.0f;
    for (int kt = wave; kt < ntiles; kt += kPfWaves) {
        tile(kt, scv, vs, false);
        float mt = scv[0];
#pragma unroll
        for (int r = 1; r < 16; r++) mt = fmaxf(mt, scv[r]);
        const float m_new = fmaxf(m_run, mt);
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) sum += exp_f<false>(scv[r] - m_new);
        l_run = l_run * exp_f<false>(m_run - m_new) + sum;
        m_run = m_new;
    }
    {
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

    // ---- pass 2: row maximum of p' = p * V_s[key] ----
    float pm = 0.0f;
    for (int kt = wave; kt < ntiles; kt += kPfWaves) {
        tile(kt, scv, vs, true);
#pragma unroll
        for (int r = 0; r < 16; r++) pm = fmaxf(pm, exp_f<false>(scv[r] - mx) * cd * vs[r]);          // masked keys give exactly 0
    }
    pm = fmaxf(pm, lane_xor_f<32>(pm));
    if (g == 0) lds_pm[wave][col] = pm;
    __syncthreads();
    float pmax = lds_pm[0][col];
#pragma unroll
    for (int w = 1; w < kPfWaves; w++) pmax = fmaxf(pmax, lds_pm[w][col]);
    const float sp = sym_scale(pmax, 127.0f);
    if (wave == 0 && g == 0) {
        lds_sp[col] = sp;
        if (p_s_out) p_s_out[(size_t)query * q_heads + h] = sp;
    }

    // ---- pass 3: probabilities, partial P.V over this wave's tiles ----
    i32x16 oacc0 = zero16(), oacc1 = zero16();
    int8_t* const prow = kStoreP ? p8_out + ((size_t)h * s + query) * s + 16 * g : nullptr;
    for (int kt = wave; kt < ntiles; kt += kPfWaves) {
        const int k0 = kt * kPfTile;
        const int8_t* vblk = vc + v_index(kvh, k0, 0, max_pos) + 16 * g;
        const i32x4 vf0 = *reinterpret_cast<const i32x4*>(vblk + (size_t)col * kVBlock);
        const i32x4 vf1 = *reinterpret_cast<const i32x4*>(vblk + (size_t)(col + 32) * kVBlock);
        tile(kt, scv, vs, true);
        i32x4 pf;
#pragma unroll
        for (int a = 0; a < 4; a++) {
            float f[4];
#pragma unroll
            for (int b = 0; b < 4; b++) f[b] = exp_f<false>(scv[4 * a + b] - mx) * cd * vs[4 * a + b];
            int nq[4];
            quant_vector(f, sp, nq);                                       // 0..127 by construction of sp
            pf[a] = (int)pack4_i8(nq[0], nq[1], nq[2], nq[3]);
        }
        if constexpr (kStoreP) *reinterpret_cast<i32x4*>(prow + k0) = pf;
        oacc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(pf, vf0, oacc0, 0, 0, 0);
        oacc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(pf, vf1, oacc1, 0, 0, 0);
    }
    if (wave < ntiles) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            atomicAdd(&lds_acc[lane][r], oacc0[r]);
            atomicAdd(&lds_acc[lane][16 + r], oacc1[r]);
        }
    }
    __syncthreads();
    const float vch0 = sc.v_ch_s ? sc.v_ch_s[kvh * kHd + col] : 1.0f, vch1 = sc.v_ch_s ? sc.v_ch_s[kvh * kHd + col + 32] : 1.0f;
#pragma unroll
    for (int rr = 0; rr < 16 / kPfWaves; rr++) {              // accumulator register r holds query row 8a + 4g + b, channel col
        const int r = wave * (16 / kPfWaves) + rr;
        const int qi = (r >> 2) * 8 + g * 4 + (r & 3);
        float* orow = o + ((size_t)(it.q0 + qi) * q_heads + h) * kHd;
        const float spq = lds_sp[qi];
        const float t0 = (float)lds_acc[lane][r] * spq, t1 = (float)lds_acc[lane][16 + r] * spq;
        orow[col] = sc.v_ch_s ? t0 * vch0 : t0;
        orow[col + 32] = sc.v_ch_s ? t1 * vch1 : t1;
    }
}

// Rows of at most kPfWaves * kPfCachedTiles * 32 = 1024 keys: the structure of pf_attention_cached_kernel.  Every score
// tile of a wave stays in registers through all the row-wide steps, so each score is formed once and each exponential
// is taken once: scores (kept) and their maximum; exponentials with the final maximum (in place) and their sum;
// p' = e * (1/sum) * V_s[key] (in place) and its maximum; rounding and P.V.  The K rows are loaded in the permuted order
// of attn_prefill.h, which makes a lane's 16 values 16 consecutive keys: their K and V scales are four 16-byte reads
// from a per-workgroup table in LDS (the scales of the row block's keys, staged once), the probability bytes leave as
// one 16-byte store, and V's operand is one 16-byte load per channel.  round(p' / s_p) goes through the reciprocal with
// the IEEE division only next to a rounding tie (quant_vector), like the per-row quantisers.
template <bool kStoreP>
static __global__ __launch_bounds__(64 * kPfWaves, 2) void pf_attention_dyn_cached_kernel(
    const int8_t* __restrict__ q8, const int8_t* __restrict__ kc, const int8_t* __restrict__ vc, DynScales sc,
    float* __restrict__ o, int8_t* __restrict__ p8_out, float* __restrict__ p_s_out, int s, int q_heads, int kv_heads,
    int max_pos, int period) {
    __shared__ float lds_m[kPfWaves][32], lds_l[kPfWaves][32], lds_pm[kPfWaves][32], lds_sp[32];
    __shared__ int lds_acc[64][33];            // [lane][16 acc0 | 16 acc1], odd pitch against bank conflicts
    __shared__ __attribute__((aligned(16))) float lds_ks[kPfWaves * kPfCachedTiles * kPfTile], lds_vs[kPfWaves * kPfCachedTiles * kPfTile];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int group = q_heads / kv_heads;
    const PfItem it = pf_item(s, q_heads, group, period);
    const int col = it.col, g = it.g, query = it.query, ntiles = it.ntiles, kvh = it.kvh, h = it.h;   // ntiles <= 32 (launcher)
    const float sq = sc.q_s[(size_t)query * q_heads + h] / sc.q_div;

    const int8_t* qrow = q8 + ((size_t)query * q_heads + h) * kHd;
    const i32x4 qf0 = *reinterpret_cast<const i32x4*>(qrow + g * 16);
    const i32x4 qf1 = *reinterpret_cast<const i32x4*>(qrow + 32 + g * 16);
    const int krow_in_tile = pf_key_of_row(col);
    // the K rows of all of this wave's tiles are requested at once
    i32x4 kf[kPfCachedTiles][2];
#pragma unroll
    for (int i = 0; i < kPfCachedTiles; i++)
        if (wave + kPfWaves * i < ntiles) {
            const int8_t* krow = kc + k_index(kvh, (wave + kPfWaves * i) * kPfTile + krow_in_tile, max_pos);
            kf[i][0] = *reinterpret_cast<const i32x4*>(krow + g * 16);
            kf[i][1] = *reinterpret_cast<const i32x4*>(krow + 32 + g * 16);
        }
    for (int j = threadIdx.x; j < ntiles * kPfTile; j += 64 * kPfWaves) {
        lds_ks[j] = sc.k_s[(size_t)j * kv_heads + kvh];
        lds_vs[j] = sc.v_s[(size_t)j * kv_heads + kvh];
    }
    for (int i = threadIdx.x; i < 64 * 33; i += 64 * kPfWaves) (&lds_acc[0][0])[i] = 0;
    __syncthreads();

    // ---- scores of this wave's tiles (kept), row maximum: register r of a lane is key k0 + 16 g + r ----
    float sv[kPfCachedTiles][16];
    float m_run = -1e32f;
#pragma unroll
    for (int i = 0; i < kPfCachedTiles; i++) {
        const int kt = wave + kPfWaves * i;
        if (kt < ntiles) {
            i32x16 acc = zero16();
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[i][0], qf0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[i][1], qf1, acc, 0, 0, 0);
            const int key0 = kt * kPfTile + 16 * g;
#pragma unroll
            for (int a = 0; a < 4; a++) {
                const float4 ks4 = *reinterpret_cast<const float4*>(&lds_ks[key0 + 4 * a]);
                const float ks[4] = {ks4.x, ks4.y, ks4.z, ks4.w};
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const float v = (float)acc[4 * a + b] * sq * ks[b];
                    sv[i][4 * a + b] = (key0 + 4 * a + b <= query) ? v : -1e32f;
                    m_run = fmaxf(m_run, sv[i][4 * a + b]);
                }
            }
        }
    }
    m_run = fmaxf(m_run, lane_xor_f<32>(m_run));
    if (g == 0) lds_m[wave][col] = m_run;
    __syncthreads();
    float mx = lds_m[0][col];
#pragma unroll
    for (int w = 1; w < kPfWaves; w++) mx = fmaxf(mx, lds_m[w][col]);
    // ---- exponentials (in place) and their sum ----
    float l_run = 0.0f;
#pragma unroll
    for (int i = 0; i < kPfCachedTiles; i++)
        if (wave + kPfWaves * i < ntiles) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                sv[i][r] = exp_f<false>(sv[i][r] - mx);                 // masked keys give exactly 0
                l_run += sv[i][r];
            }
        }
    l_run = l_run + lane_xor_f<32>(l_run);
    if (g == 0) lds_l[wave][col] = l_run;
    __syncthreads();
    float total = lds_l[0][col];
#pragma unroll
    for (int w = 1; w < kPfWaves; w++) total += lds_l[w][col];
    const float cd = 1.0f / total;
    // ---- p' = p * V_s[key] (in place) and its maximum ----
    float pm = 0.0f;
#pragma unroll
    for (int i = 0; i < kPfCachedTiles; i++) {
        const int kt = wave + kPfWaves * i;
        if (kt < ntiles) {
            const int key0 = kt * kPfTile + 16 * g;
#pragma unroll
            for (int a = 0; a < 4; a++) {
                const float4 vs4 = *reinterpret_cast<const float4*>(&lds_vs[key0 + 4 * a]);
                const float vs[4] = {vs4.x, vs4.y, vs4.z, vs4.w};
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    sv[i][4 * a + b] = sv[i][4 * a + b] * cd * vs[b];
                    pm = fmaxf(pm, sv[i][4 * a + b]);
                }
            }
        }
    }
    pm = fmaxf(pm, lane_xor_f<32>(pm));
    if (g == 0) lds_pm[wave][col] = pm;
    __syncthreads();
    float pmax = lds_pm[0][col];
#pragma unroll
    for (int w = 1; w < kPfWaves; w++) pmax = fmaxf(pmax, lds_pm[w][col]);
    const float sp = sym_scale(pmax, 127.0f);
    if (wave == 0 && g == 0) {
        lds_sp[col] = sp;
        if (p_s_out) p_s_out[(size_t)query * q_heads + h] = sp;
    }
    // ---- probabilities, partial P.V over this wave's tiles ----
    i32x16 oacc0 = zero16(), oacc1 = zero16();
    int8_t* const prow = kStoreP ? p8_out + ((size_t)h * s + query) * s + 16 * g : nullptr;
#pragma unroll
    for (int i = 0; i < kPfCachedTiles; i++) {
        const int kt = wave + kPfWaves * i;
        if (kt < ntiles) {
            const int k0 = kt * kPfTile;
            const int8_t* vblk = vc + v_index(kvh, k0, 0, max_pos) + 16 * g;
            const i32x4 vf0 = *reinterpret_cast<const i32x4*>(vblk + (size_t)col * kVBlock);
            const i32x4 vf1 = *reinterpret_cast<const i32x4*>(vblk + (size_t)(col + 32) * kVBlock);
            i32x4 pf;
#pragma unroll
            for (int a = 0; a < 4; a++) {
                const float f[4] = {sv[i][4 * a], sv[i][4 * a + 1], sv[i][4 * a + 2], sv[i][4 * a + 3]};
                int nq[4];
                quant_vector(f, sp, nq);                                   // 0..127 by construction of sp
                pf[a] = (int)pack4_i8(nq[0], nq[1], nq[2], nq[3]);
            }
            if constexpr (kStoreP) *reinterpret_cast<i32x4*>(prow + k0) = pf;
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
    }
    __syncthreads();
    const float vch0 = sc.v_ch_s ? sc.v_ch_s[kvh * kHd + col] : 1.0f, vch1 = sc.v_ch_s ? sc.v_ch_s[kvh * kHd + col + 32] : 1.0f;
#pragma unroll
    for (int rr = 0; rr < 16 / kPfWaves; rr++) {              // accumulator register r holds query row 8a + 4g + b, channel col
        const int r = wave * (16 / kPfWaves) + rr;
        const int qi = (r >> 2) * 8 + g * 4 + (r & 3);
        float* orow = o + ((size_t)(it.q0 + qi) * q_heads + h) * kHd;
        const float spq = lds_sp[qi];
        const float t0 = (float)lds_acc[lane][r] * spq, t1 = (float)lds_acc[lane][16 + r] * spq;
        orow[col] = sc.v_ch_s ? t0 * vch0 : t0;
        orow[col + 32] = sc.v_ch_s ? t1 * vch1 : t1;
    }
}

// ---- decode: chunked kernels (one workgroup per (kv head, 128-key chunk), wave g = query head kvh*group+g) -------------
static __global__ __launch_bounds__(256) void dec_scores_dyn_kernel(const int8_t* __restrict__ q8, const int8_t* __restrict__ kc,
                                                                    DynScales sc, float* __restrict__ scores,
                                                                    float2* __restrict__ stats, int32_t* __restrict__ o_acc,
                                                                    int len, int group, int kv_heads, int max_pos) {
    const int chunk = blockIdx.x, kvh = blockIdx.y;
    const int g = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int qh = kvh * group + g;
    if (chunk == 0) o_acc[qh * kHd + lane] = 0;
    const i32x4* qv = reinterpret_cast<const i32x4*>(q8 + (size_t)qh * kHd);
    const i32x4 q0 = qv[0], q1 = qv[1], q2 = qv[2], q3 = qv[3];
    const float sq = sc.q_s[qh] / sc.q_div;
    float scv[kChunk / 64];
    float mx = -1e32f;
#pragma unroll
    for (int j = 0; j < kChunk / 64; j++) {
        const int pos = chunk * kChunk + j * 64 + lane;
        scv[j] = -1e32f;
        if (pos < len) {
            const i32x4* kr = reinterpret_cast<const i32x4*>(kc + k_index(kvh, pos, max_pos));
            int acc = dot16(kr[0], q0, 0);
            acc = dot16(kr[1], q1, acc);
            acc = dot16(kr[2], q2, acc);
            acc = dot16(kr[3], q3, acc);
            scv[j] = (float)acc * sq * sc.k_s[(size_t)pos * kv_heads + kvh];
            scores[(size_t)qh * len + pos] = scv[j];
            mx = fmaxf(mx, scv[j]);
        }
    }
    mx = wave_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < kChunk / 64; j++)
        if (chunk * kChunk + j * 64 + lane < len) sum += exp_f(scv[j] - mx);
    sum = wave_sum(sum);
    if (lane == 0) stats[qh * kMaxChunks + chunk] = make_float2(mx, sum);
}

__device__ __forceinline__ void dyn_row_stats(const float2* stats, int qh, int nchunks, int lane, float& mx, float& cd) {
    float m_c = -1e32f, l_c = 0.0f;
    if (lane < nchunks) { const float2 st = stats[qh * kMaxChunks + lane]; m_c = st.x; l_c = st.y; }
    mx = wave_max(m_c);
    const float sum = wave_sum(lane < nchunks ? l_c * exp_f(m_c - mx) : 0.0f);
    cd = 1.0f / sum;
}

// scores -> p' = p * V_s[key] in place; chunk maximum of p'
static __global__ __launch_bounds__(256) void dec_pmax_dyn_kernel(float* __restrict__ scores, const float2* __restrict__ stats,
                                                                  DynScales sc, float* __restrict__ pmax, int len, int group,
                                                                  int kv_heads) {
    const int nchunks = (len + kChunk - 1) / kChunk;
    const int chunk = blockIdx.x, kvh = blockIdx.y;
    const int g = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int qh = kvh * group + g;
    float mx, cd;
    dyn_row_stats(stats, qh, nchunks, lane, mx, cd);
    float pm = 0.0f;
#pragma unroll
    for (int j = 0; j < kChunk / 64; j++) {
        const int pos = chunk * kChunk + j * 64 + lane;
        if (pos < len) {
            const float pp = exp_f(scores[(size_t)qh * len + pos] - mx) * cd * sc.v_s[(size_t)pos * kv_heads + kvh];
            scores[(size_t)qh * len + pos] = pp;
            pm = fmaxf(pm, pp);
        }
    }
    pm = wave_max(pm);
    if (lane == 0) pmax[qh * kMaxChunks + chunk] = pm;
}

static __global__ __launch_bounds__(256) void dec_pv_dyn_kernel(const float* __restrict__ pp, const float* __restrict__ pmax,
                                                                const int8_t* __restrict__ vc, int32_t* __restrict__ o_acc,
                                                                int8_t* __restrict__ p8_out, float* __restrict__ p_s, int len,
                                                                int group, int max_pos) {
    __shared__ uint32_t p_lds[4][kChunk / 4];
    const int nchunks = (len + kChunk - 1) / kChunk;
    const int chunk = blockIdx.x, kvh = blockIdx.y;
    const int g = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int qh = kvh * group + g;
    const float sp = sym_scale(wave_max(lane < nchunks ? pmax[qh * kMaxChunks + lane] : 0.0f), 127.0f);
    if (chunk == 0 && lane == 0) p_s[qh] = sp;
    int8_t* pb = reinterpret_cast<int8_t*>(p_lds[g]);
#pragma unroll
    for (int j = 0; j < kChunk / 64; j++) {
        const int pos = chunk * kChunk + j * 64 + lane;
        int p8 = 0;
        if (pos < len) {
            p8 = (int)roundf(pp[(size_t)qh * len + pos] / sp);
            if (p8_out) p8_out[(size_t)qh * len + pos] = (int8_t)p8;
        }
        pb[j * 64 + lane] = (int8_t)p8;
    }
    __syncthreads();
    int acc = 0;
#pragma unroll
    for (int j = 0; j < kChunk / 64; j++) {
        const int pos_blk = chunk * kChunk + j * 64;
        if (pos_blk < len) {
            const i32x4* vr = reinterpret_cast<const i32x4*>(vc + v_index(kvh, pos_blk, lane, max_pos));
            const i32x4* pr = reinterpret_cast<const i32x4*>(p_lds[g] + j * 16);
#pragma unroll
            for (int c = 0; c < 4; c++) acc = dot16(pr[c], vr[c], acc);
        }
    }
    atomicAdd(&o_acc[qh * kHd + lane], acc);
}

static __global__ __launch_bounds__(256) void dec_out_dyn_kernel(const int32_t* __restrict__ o_acc, const float* __restrict__ p_s,
                                                                 const float* __restrict__ v_ch_s, float* __restrict__ o, int n,
                                                                 int group) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const int qh = i / kHd;
        const float t = (float)o_acc[i] * p_s[qh];
        o[i] = v_ch_s ? t * v_ch_s[(qh / group) * kHd + i % kHd] : t;
    }
}

// scratch of the decode entry point: the calling stream's buffer (stream_scratch), carved into its arrays
struct DynScratch {
    float* scores = nullptr;
    float2* stats = nullptr;
    float* pmax = nullptr;
    float* p_s = nullptr;
    int32_t* o_acc = nullptr;
};

static int dyn_scratch_of_stream(hipStream_t st, int q_heads, int len, DynScratch* out) {
    const size_t heads = q_heads > 32 ? q_heads : 32;
    const size_t need = (size_t)q_heads * len;
    const size_t elems = need > heads * 4096 ? need : heads * 4096;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t b_scores = up(elems * sizeof(float)), b_stats = up(heads * kMaxChunks * sizeof(float2)),
                 b_pmax = up(heads * kMaxChunks * sizeof(float)), b_ps = up(heads * sizeof(float)), b_acc = up(heads * kHd * sizeof(int32_t));
    void* base = nullptr;
    int rc = stream_scratch(kScratchMhaDecodeDyn, st, b_scores + b_stats + b_pmax + b_ps + b_acc, &base);
    if (rc) return rc;
    char* p = static_cast<char*>(base);
    out->scores = reinterpret_cast<float*>(p); p += b_scores;
    out->stats = reinterpret_cast<float2*>(p); p += b_stats;
    out->pmax = reinterpret_cast<float*>(p); p += b_pmax;
    out->p_s = reinterpret_cast<float*>(p); p += b_ps;
    out->o_acc = reinterpret_cast<int32_t*>(p);
    return FLEXLLM_OK;
}

}  // namespace fx

using namespace fx;

extern "C" {

int flexllm_mha_i8_prefill_dyn(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache, const flexllm_mha_dyn_scales* sc,
                               float* o, int8_t* p8_out, float* p_s_out, int s, int q_heads, int kv_heads, int head_dim,
                               int max_pos, void* stream) {
    FX_REQUIRE(q8 && k_cache && v_cache && sc && o, "mha_prefill_dyn: null pointer");
    FX_REQUIRE(sc->q_s && sc->k_s && sc->v_s, "mha_prefill_dyn: null scale array");
    FX_REQUIRE(sc->q_scale_div > 0.0f, "mha_prefill_dyn: q_scale_div=%g must be positive", (double)sc->q_scale_div);
    FX_REQUIRE(head_dim == kHd, "mha_prefill_dyn: head_dim=%d (only 64)", head_dim);
    FX_REQUIRE(kv_heads > 0 && q_heads % kv_heads == 0, "mha_prefill_dyn: q_heads=%d kv_heads=%d", q_heads, kv_heads);
    FX_REQUIRE(s > 0 && s % kPfTile == 0 && s <= max_pos && max_pos % kVBlock == 0,
               "mha_prefill_dyn: s=%d max_pos=%d (s a positive multiple of 32, s <= max_pos, max_pos %% 64 == 0)", s, max_pos);
    int dev = 0, n_cu = 0;
    FX_HIP(hipGetDevice(&dev));
    FX_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    if (n_cu <= 0) n_cu = 256;
    const DynScales d = {sc->q_s, sc->k_s, sc->v_s, sc->v_ch_s, sc->q_scale_div};
    const int grid = (s / kPfTile) * q_heads;
    if (s <= kPfWaves * kPfCachedTiles * kPfTile) {            // every row fits the registers of eight waves
        if (p8_out)
            pf_attention_dyn_cached_kernel<true><<<grid, 64 * kPfWaves, 0, as_stream(stream)>>>(q8, k_cache, v_cache, d, o, p8_out, p_s_out, s,
                                                                                                q_heads, kv_heads, max_pos, n_cu);
        else
            pf_attention_dyn_cached_kernel<false><<<grid, 64 * kPfWaves, 0, as_stream(stream)>>>(q8, k_cache, v_cache, d, o, nullptr, p_s_out, s,
                                                                                                 q_heads, kv_heads, max_pos, n_cu);
    } else if (p8_out) {
        pf_attention_dyn_kernel<true><<<grid, 64 * kPfWaves, 0, as_stream(stream)>>>(q8, k_cache, v_cache, d, o, p8_out, p_s_out, s, q_heads,
                                                                                     kv_heads, max_pos, n_cu);
    } else {
        pf_attention_dyn_kernel<false><<<grid, 64 * kPfWaves, 0, as_stream(stream)>>>(q8, k_cache, v_cache, d, o, nullptr, p_s_out, s, q_heads,
                                                                                      kv_heads, max_pos, n_cu);
    }
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_mha_i8_decode_dyn(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache, const flexllm_mha_dyn_scales* sc,
                              float* o, int8_t* p8_out, float* p_s_out, int len, int q_heads, int kv_heads, int head_dim,
                              int max_pos, void* stream) {
    FX_REQUIRE(q8 && k_cache && v_cache && sc && o, "mha_decode_dyn: null pointer");
    FX_REQUIRE(sc->q_s && sc->k_s && sc->v_s, "mha_decode_dyn: null scale array");
    FX_REQUIRE(sc->q_scale_div > 0.0f, "mha_decode_dyn: q_scale_div=%g must be positive", (double)sc->q_scale_div);
    FX_REQUIRE(head_dim == kHd, "mha_decode_dyn: head_dim=%d (only 64)", head_dim);
    FX_REQUIRE(kv_heads > 0 && q_heads % kv_heads == 0 && q_heads / kv_heads >= 1 && q_heads / kv_heads <= 4,
               "mha_decode_dyn: q_heads=%d kv_heads=%d (group size 1..4)", q_heads, kv_heads);
    FX_REQUIRE(len >= 1 && len <= kChunk * kMaxChunks && len <= max_pos && max_pos % kVBlock == 0,
               "mha_decode_dyn: len=%d max_pos=%d (1 <= len <= 8192, len <= max_pos, max_pos %% 64 == 0)", len, max_pos);
    hipStream_t st = as_stream(stream);
    DynScratch ds;
    int rc = dyn_scratch_of_stream(st, q_heads, len, &ds);
    if (rc) return rc;
    const DynScales d = {sc->q_s, sc->k_s, sc->v_s, sc->v_ch_s, sc->q_scale_div};
    const int group = q_heads / kv_heads;
    dim3 grid((len + kChunk - 1) / kChunk, kv_heads);
    dec_scores_dyn_kernel<<<grid, 64 * group, 0, st>>>(q8, k_cache, d, ds.scores, ds.stats, ds.o_acc, len, group, kv_heads, max_pos);
    dec_pmax_dyn_kernel<<<grid, 64 * group, 0, st>>>(ds.scores, ds.stats, d, ds.pmax, len, group, kv_heads);
    float* p_s = p_s_out ? p_s_out : ds.p_s;
    dec_pv_dyn_kernel<<<grid, 64 * group, 0, st>>>(ds.scores, ds.pmax, v_cache, ds.o_acc, p8_out, p_s, len, group, max_pos);
    const int n = q_heads * kHd;
    dec_out_dyn_kernel<<<(n + 255) / 256, 256, 0, st>>>(ds.o_acc, p_s, sc->v_ch_s, o, n, group);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // extern "C"

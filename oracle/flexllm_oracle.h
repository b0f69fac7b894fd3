/*
 * CPU oracle for the FlexLLM quantized-transformer datapath.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * HLS modules, used as the checker by tests/, by the smoke run and as the timed
 * CPU baseline of the benchmark.  Nothing in the shipped library links, calls
 * or falls back to it.
 *
 * Conventions: every tensor is a dense row-major array, token-major
 * (x[token][feature]); the reference's stream packing ([token block][feature]
 * [token lane] for prefill, block-partitioned lanes for decode) is a pure
 * permutation restated separately in fxo_pack_* / fxo_unpack_*.
 * All float arithmetic is IEEE binary32 with no contraction (build with
 * -ffp-contract=off) and follows the reference's operation order where the
 * order is observable in the result.
 *
 * Parity pinning (what independently checks each restatement) is listed per
 * function; "unpinned" means only the restated formula itself is available.
 */
#ifndef FLEXLLM_ORACLE_H
#define FLEXLLM_ORACLE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Number of OpenMP threads for the loops over independent outputs (n <= 0: all processors).  Results do not depend
 * on it. */
void fxo_set_threads(int n);
int fxo_max_threads(void);

/* ---- quant.h ------------------------------------------------------------ */
/* Modules/quant.h:6-112 (prefill) and :332-431 (decode), symmetric branch.
 * Pinned by: absmax element maps to +-(2^(b-1)-1), all-zero row gives s=1,
 * ties round away from zero, brute-force numpy float32 restatement. */
void fxo_quant_sym(const float* x, int rows, int dim, int bits, int8_t* q, float* s);
/* Same functions, asymmetric branch (:53-82, :382-405): s=(max-min)/(2^b-1), b=min. */
void fxo_quant_asym(const float* x, int rows, int dim, int bits, uint8_t* q, float* s, float* b);
/* Modules/quant.h:115-164, :434-524: y=(float(acc)*s_x)*s_w [+ b_x*sum_w]. b_x/w_sum may be NULL. */
void fxo_dequant(const int32_t* acc, int rows, int n, const float* s_x, const float* b_x,
                 const float* w_s, const float* w_sum, float* y);
/* Modules/quant.h:252-293, :716-755: q=clamp(round(x/(factor*scale[h]))); x is [rows][heads][dim].
 * is_signed: clamp to [-2^(b-1), 2^(b-1)-1]; else clamp high only to 2^b-1 and store the low 8 bits. */
void fxo_static_quant(const float* x, int rows, int heads, int dim, const float* scale,
                      float factor, int is_signed, int bits, int8_t* q);
/* Modules/quant.h:296-326, :758-805: y=(float(acc)*a_s[ah])*w_s[ah/(act_heads/w_heads)]; acc is [rows][act_heads][dim]. */
void fxo_static_dequant(const int32_t* acc, int rows, int act_heads, int w_heads, int dim,
                        const float* a_s, const float* w_s, float* y);
/* Modules/quant.h:527-617: dynamic per-(token,head) symmetric quant; x is [rows][heads][dim], s is [rows][heads]. */
void fxo_head_quant_sym(const float* x, int rows, int heads, int dim, int bits, int8_t* q, float* s);

/* ---- Linear_Layer.h / PE.h / MHA.h systolic arrays ------------------------ */
/* C[m][n] = sum_k A[m][k]*W[n][k], exact.  Modules/Linear_Layer.h:293-341, :862-923 with the
 * i8 PEs of Modules/PE.h:482-583; golden loop SpinQuant_Llama_32_1B/Linear_Layer_Decoding_tb.cpp:60-67. */
void fxo_linear_i8(const int8_t* a, const int8_t* w, int m, int k, int n, int32_t* c);
/* Same with unsigned activations (is_uint_input=true). */
void fxo_linear_u8i8(const uint8_t* a, const int8_t* w, int m, int k, int n, int32_t* c);

/* ---- FHT.h ---------------------------------------------------------------- */
/* Modules/FHT.h:7-67 / :69-129: log2(n) x (perfect shuffle, adjacent butterfly), then / scale.
 * Pinned by: explicit Sylvester matrix (n<=64, exact on small integers), involution, Parseval. */
void fxo_fht(const float* x, int rows, int n, float scale, float* y);

/* ---- LayerNorm.h ---------------------------------------------------------- */
/* Modules/LayerNorm.h:28-183 non-versal: four partial sums by k%4. */
void fxo_rmsnorm_pref(const float* x, const float* gamma, int rows, int dim, float eps, float* y);
/* Modules/LayerNorm.h:210-310 non-versal: per-lane k%4 partials, lanes summed in order.
 * Lane i holds features [i*dim/bp, (i+1)*dim/bp). */
void fxo_rmsnorm_dec(const float* x, const float* gamma, int dim, int block_parallel, float eps, float* y);

/* ---- RoPE.h --------------------------------------------------------------- */
/* Table per the formula kept in Modules/RoPE.h:28-50 (Llama-3 frequency scaling). tables are [max_pos][head_dim/2]. */
void fxo_rope_table(int max_pos, int head_dim, float theta, int factor, int low_freq_factor,
                    int high_freq_factor, int original_max_pe, float* sin_t, float* cos_t);
/* Modules/RoPE.h:8-94, :96-173: rotate-half; x is [tokens][heads][head_dim], token t is at position pos0+t. */
void fxo_rope(const float* x, int tokens, int heads, int head_dim, const float* sin_t,
              const float* cos_t, int pos0, float* y);

/* ---- Swish.h / Linear_Layer.h gate / Residual_Layer.h ---------------------- */
void fxo_swish(const float* x, int n, float* y);                    /* Modules/Swish.h:5-41 */
void fxo_gate(const float* a, const float* b, int n, float* y);     /* Modules/Linear_Layer.h:612-630, :1103-1121 */
void fxo_residual(const float* a, const float* b, int n, float* y); /* Modules/Residual_Layer.h:47-87 */

/* ---- Softmax.h / MHA.h ---------------------------------------------------- */
/* Modules/Softmax.h:6-163 and :456-635 (non-versal, enable_sub_max, no scale); ragged dim allowed. */
void fxo_softmax(const float* x, int rows, int dim, float* y);
/* Softmax.h:262-360 dec_Softmax on a block-partitioned vector, optional division of the exponent by `scale` */
void fxo_softmax_dec(const float* x, int dim, int bp, int enable_scale, float scale, float* y);
/* Linear_Layer.h:1041-1100 + PE.h:709-752: fp32 GEMV, four partial sums by k % 4 */
void fxo_linear_f32(const float* x, const float* w, int k, int n, float* y);
/* HMT.h:278-316: scores over all memory slots, scaled softmax, weighted sum of the memories (mem_num <= 1024) */
void fxo_hmt_retrieve(const float* q, const float* kmem, const float* mmem, int mem_num, int hidden, int bp,
                      float scale, float* a_sft, float* p_out);
/* Modules/MHA.h:246-273: y[q][k] = k<=q ? x : -1e32 ; x is [rows][heads][dim]. */
void fxo_causal_mask(const float* x, int rows, int heads, int dim, float* y);

/* Attention scale tables for one layer (static per-head scales of the shipped graphs). */
typedef struct {
    const float* q_s; /* [q_heads]  */
    const float* k_s; /* [kv_heads] */
    const float* v_s; /* [kv_heads] */
    const float* a_s; /* [q_heads]  */
} fxo_mha_scales;

/* Whole prefill attention of SpinQuant_Llama_32_1B/MHA_i8xi8.h:369-427 for one layer.
 * q [s][q_heads][64], k,v [s][kv_heads][64] fp32 (post-RoPE). Outputs (any may be NULL):
 * q8,k8,v8 int8 tensors, p8 [q_heads][s][s] uint8, o [s][q_heads][64] fp32. */
void fxo_mha_prefill(const float* q, const float* k, const float* v, int s, int q_heads, int kv_heads,
                     int head_dim, const fxo_mha_scales* sc, int8_t* q8, int8_t* k8, int8_t* v8,
                     uint8_t* p8, float* o);
/* The same attention from the int8 tensors (q8 [s][q_heads][64], k8, v8 [s][kv_heads][64]); with p8_in the given
 * probability bytes [q_heads][s][s] take the place of the computed ones in P.V (fxo_mha_prefill is the static
 * quantisation followed by this function, so the checks that pin one pin the other). */
void fxo_mha_prefill_i8(const int8_t* q8, const int8_t* k8, const int8_t* v8, int s, int q_heads, int kv_heads,
                        int head_dim, const fxo_mha_scales* sc, const uint8_t* p8_in, uint8_t* p8_out, float* o);
/* Decode attention of MHA_i8xi8.h:1027-1114 for one layer, one query against len cached keys
 * (the new token's k/v already appended). q8 [q_heads][64], caches [len][kv_heads][64]. */
void fxo_mha_decode(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache, int len,
                    int q_heads, int kv_heads, int head_dim, const fxo_mha_scales* sc,
                    uint8_t* p8, float* o);

/* Attention with DYNAMIC per-(token, head) scales, the library's own quantiser (Modules/quant.h:527-617,
 * dec_MHA_quant_layer_fp32_qint<8,false>: s = absmax/127, 0 -> 1) applied to Q, K, V and to the probabilities, with the
 * per-token scale streams of Modules/quant.h:165-246 (pref_static_sym_quant/dequant_layer: score = acc * s_q[token] *
 * s_k[key]) and the K scale cache of Modules/MHA.h:9-71, :393-445.
 *   q8, s_q = quant(q[t][h]);  Q_s = s_q / sqrt(head_dim)   (the factor the static path folds into Q's scale)
 *   k8, K_s[t][kvh];  v8, V_s[t][kvh]
 *   a[i][j] = (float(q8_i . k8_j) * Q_s[i][h]) * K_s[j][kvh];  causal mask -1e32;  softmax (Softmax.h)
 *   p'[j] = p[j] * V_s[j][kvh]      V's per-token scale varies along the reduction of P.V, so it is folded into the
 *                                    probabilities before they are quantised (the reference library keeps V's scale
 *                                    per channel and static, Modules/MHA.h:713-738, and has no per-token V path)
 *   P8, s_p = quant(p')              int8 in 0..127, one scale per (query, head)
 *   o[i][h][d] = float(sum_j P8[j] * v8[j][d]) * s_p  (* v_ch_s[kvh][d] when a per-channel V scale is given)
 * Outputs (any may be NULL): q8 [s][qh][hd], q_s [s][qh] (= Q_s), k8/v8 [s][kvh][hd], k_s/v_s [s][kvh],
 * p8 [qh][s][s] int8, p_s [s][qh], o [s][qh][hd].  v_ch_s: optional [kvh][hd] input.
 * Pinned by: float64 fake-quant golden built like MHA_i8xi8_prefilling_tb.cpp:26-218 with per-token scales (each
 * of the three facts above switched off once must be noticed), decode == prefill row bit for bit, the per-channel
 * factor as an exact float32 product. */
void fxo_mha_prefill_dyn(const float* q, const float* k, const float* v, int s, int q_heads, int kv_heads, int head_dim,
                         const float* v_ch_s, int8_t* q8, float* q_s, int8_t* k8, float* k_s, int8_t* v8, float* v_s,
                         int8_t* p8, float* p_s, float* o);
/* One query against len cached keys: q8 [qh][hd] with Q_s [qh]; caches [len][kvh][hd] with K_s, V_s [len][kvh]. */
void fxo_mha_decode_dyn(const int8_t* q8, const float* q_s, const int8_t* k_cache, const float* k_s,
                        const int8_t* v_cache, const float* v_s, const float* v_ch_s, int len, int q_heads,
                        int kv_heads, int head_dim, int8_t* p8, float* p_s, float* o);

/* ---- Llama-3.2-1B W8A8 layer / model (graph order of SpinQuant_Prefilling.h:940-1049 and
 *      SpinQuant_Decoding_mem_opt.h:1050-1126 with int8 symmetric linear layers) ---- */
typedef struct {
    int layers, hidden, kv_hidden, inter, q_heads, kv_heads, head_dim, vocab, max_pos;
    float eps, fht_scale;
    /* per layer l: int8 row-major [N][K] weights and fp32 per-channel scales */
    const int8_t* const* wq; const int8_t* const* wk; const int8_t* const* wv; const int8_t* const* wo;
    const int8_t* const* wg; const int8_t* const* wu; const int8_t* const* wd;
    const float* const* sq; const float* const* sk; const float* const* sv; const float* const* so;
    const float* const* sg; const float* const* su; const float* const* sd;
    const float* gamma;     /* [2*layers+1][hidden] */
    const float* q_s; const float* k_s; const float* v_s; const float* a_s; /* [layers][heads] */
    const float* rope_sin; const float* rope_cos; /* [max_pos][head_dim/2] */
    const uint16_t* embed;  /* fp16 [vocab][hidden], tied lm_head */
} fxo_model;

/* One token through all layers at position pos; caches are [layer][max_pos][kv_hidden] int8.
 * x_in fp32[hidden]; writes logits fp32[vocab] (NULL to skip) and hidden_out fp32[hidden] (pre final norm). */
void fxo_llama_decode_token(const fxo_model* m, const float* x_in, int pos, int8_t* k_cache,
                            int8_t* v_cache, float* hidden_out, float* logits);
/* Prefill s tokens (positions 0..s-1). x_in [s][hidden]; fills caches; hidden_out [s][hidden]. */
void fxo_llama_prefill(const fxo_model* m, const float* x_in, int s, int8_t* k_cache, int8_t* v_cache,
                       float* hidden_out);
/* fp16 helpers + lm_head: logits[v] = sum_k fp16(E[v][k]) * n[k], sequential fp32 accumulation. */
float fxo_half_to_float(uint16_t h);
void fxo_embed(const uint16_t* table, int hidden, int token, float* y);
void fxo_lm_head(const uint16_t* table, int vocab, int hidden, const float* n, float* logits);
/* Logits.h:145-279 top-k sampling (see the .c file for the exact correspondence); returns the sampled token id */
int fxo_sample_topk(const float* logits, int n, int top_k, int lanes, float rand_seed, int enable_sub_max,
                    int* top_idx, float* top_val, float* top_prob);
int fxo_argmax(const float* x, int n);

/* ---- data_io.h layouts ----------------------------------------------------- */
/* Modules/data_io.h:6-38: prefill buffers are [token/tp][feature][token%tp]. */
void fxo_pack_pref(const float* x, int tokens, int dim, int tp, float* packed);
void fxo_unpack_pref(const float* packed, int tokens, int dim, int tp, float* x);
/* Modules/data_io.h:348-387: decode buffers are [feature % (dim/bp)][feature / (dim/bp)]. */
void fxo_pack_dec(const float* x, int dim, int bp, float* packed);
void fxo_unpack_dec(const float* packed, int dim, int bp, float* x);

#ifdef __cplusplus
}
#endif
#endif

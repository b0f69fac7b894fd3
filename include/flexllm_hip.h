/*
 * flexllm_hip.h - C ABI of libflexllm_hip.so: the FlexLLM quantized-transformer
 * datapath (Modules/ + MHA_i8xi8.h of Crazy-James26/FlexLLM) on one MI355X (gfx950).
 *
 * Conventions
 *  - Every tensor pointer is DEVICE memory, dense row-major, token-major
 *    (x[token][feature]); weights are int8 [out_features][in_features].
 *  - `stream` is a hipStream_t passed as void* (NULL = default stream).  Calls only
 *    enqueue work; nothing synchronises unless stated.
 *  - Return value: 0 on success, a negative FLEXLLM_E* code otherwise (the reference
 *    functions return void and print; errors here never print).  flexllm_last_error()
 *    gives the message of the last failure on the calling thread.
 *  - Integer results (int32 accumulators, int8/uint8 tensors) are bit-exact functions of
 *    their inputs.  fp32 results follow the reference's operation order except for
 *    reductions over a row (sum of squares, sum of exponentials), whose association
 *    differs; those agree to <=1e-3 relative.
 *  - Four stand-alone entry points need scratch memory beyond their arguments: flexllm_argmax_f32,
 *    flexllm_sample_topk_f32 (rows of 4096 logits and more), flexllm_mha_i8_decode and flexllm_mha_i8_decode_dyn.
 *    The library keeps one buffer per (device, stream, entry point), allocated on the first call on that stream
 *    and grown on demand (growing waits for the stream's earlier work).  Calls on different streams therefore never
 *    share scratch and may run at the same time, from one host thread or several; calls on one stream run in
 *    stream order.  flexllm_rt_stream_destroy releases a stream's buffers; buffers of streams created elsewhere
 *    live until the process ends.  A flexllm_llama object owns all of its buffers; use one object from one
 *    stream at a time.
 *
 * Reference citations are relative to the reference tree root.
 */
#ifndef FLEXLLM_HIP_H
#define FLEXLLM_HIP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define FLEXLLM_OK 0
#define FLEXLLM_EINVAL (-1)   /* bad shape / null pointer / unsupported size */
#define FLEXLLM_EHIP (-2)     /* a HIP runtime call failed */
#define FLEXLLM_ENOMEM (-3)

const char* flexllm_last_error(void);
/* Library version and the offload architecture the kernels were built for ("gfx950"). */
const char* flexllm_build_info(void);

/* ---- minimal runtime plumbing for hosts without a HIP binding (ctypes, cgo ...) ---- */
int flexllm_rt_device_count(int* count);
int flexllm_rt_device_name(char* buf, int buflen);
int flexllm_rt_malloc(void** dptr, size_t bytes);
int flexllm_rt_free(void* dptr);
/* Free and total device memory of the current device in bytes (hipMemGetInfo). */
int flexllm_rt_mem_info(size_t* free_bytes, size_t* total_bytes);
int flexllm_rt_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream);
int flexllm_rt_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream);
int flexllm_rt_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream);
int flexllm_rt_memset(void* dst, int value, size_t bytes, void* stream);
int flexllm_rt_stream_create(void** stream);
int flexllm_rt_stream_destroy(void* stream);
int flexllm_rt_stream_sync(void* stream);
int flexllm_rt_device_sync(void);
int flexllm_rt_event_create(void** event);
int flexllm_rt_event_destroy(void* event);
int flexllm_rt_event_record(void* event, void* stream);
int flexllm_rt_event_sync(void* event);
int flexllm_rt_event_elapsed_ms(void* start, void* stop, float* ms);
/* Fill with a counter-based PRNG (SplitMix64 of seed+index): int8 uniform in [lo,hi], fp32
 * uniform in [lo,hi), fp32 standard normal (Box-Muller).  Bit-identical to
 * flexllm_amd.synth on the host. */
int flexllm_rt_fill_i8(int8_t* dst, size_t n, uint64_t seed, int lo, int hi, void* stream);
int flexllm_rt_fill_uniform_f32(float* dst, size_t n, uint64_t seed, float lo, float hi, void* stream);
int flexllm_rt_fill_uniform_f16(uint16_t* dst, size_t n, uint64_t seed, float lo, float hi, void* stream);

/* ---- measurement probes (no counterpart in the reference: they exist so that a benchmark can print the rate this GPU
 *      sustains next to the published peak a roofline is priced against) ------------------------------------------- */
/* Matrix cores alone: `workgroups` x 4 waves, each issuing iters x 16 v_mfma_i32_32x32x32_i8 on a 4x4 grid of
 * accumulator tiles = workgroups * 4 * iters * 16 * 65536 int8 operations per launch.  random_operands: pseudo-random
 * operand bytes (else zeros, which draw less power and run at a higher clock); from_lds: the eight operand fragments
 * are re-read from LDS at every step, as in a GEMM's main loop (else they stay in registers).  sink: device
 * [workgroups * 256] int32 (written, keeps the work alive); clocks: optional device [2] uint64 = {shader-clock cycles,
 * 100 MHz wall-clock ticks} of one wave's loop, i.e. the shader clock under this load. */
int flexllm_probe_mfma_i8(int iters, int random_operands, int from_lds, int workgroups, int* sink, unsigned long long* clocks,
                          void* stream);
/* Read-only stream over `bytes` (a multiple of 16) of device memory with 16-byte loads (non_temporal: with the
 * non-temporal hint), contiguous 32 KiB blocks per workgroup; sink: device [workgroups * 4] uint32. */
int flexllm_probe_hbm_read(const void* src, size_t bytes, int workgroups, int non_temporal, unsigned* sink, void* stream);

/* ---- quant.h ------------------------------------------------------------------------ */
/* Per-token symmetric int8 quantisation: s=absmax/127 (0 -> 1), q=round_half_away(x/s).
 * Replaces pref_quant_layer_fp32_qint<8,false,...> (Modules/quant.h:6-112) and
 * dec_quant_layer_fp32_qint<8,false,...> (Modules/quant.h:332-431).  x [rows][dim] fp32,
 * q [rows][dim] int8, s [rows] fp32.  dim % 4 == 0. */
int flexllm_quant_sym_i8(const float* x, int8_t* q, float* s, int rows, int dim, void* stream);
/* Per-token asymmetric unsigned quantisation (bits in 2..8): s=(max-min)/(2^bits-1), b=min,
 * q=round((x-b)/s) stored one value per byte.  Modules/quant.h:53-82, :382-405. */
int flexllm_quant_asym_u8(const float* x, uint8_t* q, float* s, float* b, int bits, int rows, int dim, void* stream);
/* y[r][n] = (float(acc[r][n]) * s_x[r]) * w_s[n]  [+ b_x[r] * w_sum[n]] ; b_x and w_sum may both be NULL.
 * Replaces pref_dequant_layer_qint_fp32 (Modules/quant.h:115-164) and
 * dec_dequant_layer_qint_fp32(_bandwidth) (Modules/quant.h:434-524). */
int flexllm_dequant_i32_f32(const int32_t* acc, const float* s_x, const float* b_x, const float* w_s,
                            const float* w_sum, float* y, int rows, int n, void* stream);
/* Static per-head quantisation: q=clamp(round(x/(factor*scale[h]))); x [rows][heads][dim].
 * is_signed=1: clamp to [-128,127]; 0: clamp high to 255, stored as uint8 bit pattern.
 * Replaces pref_static_sym_per_tensor_quant_layer_fp32_qint (Modules/quant.h:252-293) and
 * dec_MHA_static_sym_per_tensor_quant_layer_fp32_qint (Modules/quant.h:716-755). */
int flexllm_static_quant_i8(const float* x, int8_t* q, const float* scale, float factor, int is_signed,
                            int rows, int heads, int dim, void* stream);
/* y=(float(acc)*a_s[h])*w_s[h/(act_heads/w_heads)]; acc [rows][act_heads][dim].
 * Replaces pref_static_sym_per_tensor_dequant_layer_qint_fp32 (Modules/quant.h:296-326) and the
 * decode form (Modules/quant.h:758-805). */
int flexllm_static_dequant_i32_f32(const int32_t* acc, float* y, const float* a_s, const float* w_s,
                                   int rows, int act_heads, int w_heads, int dim, void* stream);
/* Dynamic per-(token,head) symmetric int8 quantisation, x [rows][heads][dim], s [rows][heads].
 * Replaces dec_MHA_quant_layer_fp32_qint<8,false,...> (Modules/quant.h:527-617). */
int flexllm_head_quant_sym_i8(const float* x, int8_t* q, float* s, int rows, int heads, int dim, void* stream);

/* ---- Linear_Layer.h ------------------------------------------------------------------- */
/* Decode GEMV, exact: acc[n] = sum_k x[k]*W[n][k].  Replaces dec_Linear_Layer_i4xi4
 * (Modules/Linear_Layer.h:862-923) instantiated with the int8 PEs (Modules/PE.h:793-830,
 * Modules/MHA.h:564-611).  k % 16 == 0, k <= 16384. */
int flexllm_linear_i8_gemv(const int8_t* x, const int8_t* w, int32_t* acc, int k, int n, void* stream);
/* Fused decode linear: y[n] = (float(acc[n])*s_x[0])*w_s[n] (+ residual[n] if residual != NULL).
 * = GEMV above + dec_dequant_layer_qint_fp32_bandwidth (Modules/quant.h:470-524)
 * (+ dec_Residual_Layer, Modules/Residual_Layer.h:69-87). */
int flexllm_linear_i8_gemv_dequant(const int8_t* x, const float* s_x, const int8_t* w, const float* w_s,
                                   const float* residual, float* y, int k, int n, void* stream);
/* The whole decode linear of one token in one launch: per-token symmetric int8 quantisation of x fp32 [k] (the bytes and
 * the scale of flexllm_quant_sym_i8), GEMV, dequantisation (+ residual) - what the reference's quantised linear wrapper
 * chains per token: dec_quant_layer_fp32_qint -> dec_Linear_Layer -> dec_dequant_layer_qint_fp32_bandwidth
 * (SpinQuant_Llama_32_1B/Linear_Layer_test.h:332-364).  Optional outputs: s_x_out [1] the activation scale, q_out [k] the
 * quantised activation.  k % 16 == 0, k <= 4096. */
int flexllm_quant_linear_i8_gemv_dequant(const float* x, const int8_t* w, const float* w_s, const float* residual, float* y,
                                         float* s_x_out, int8_t* q_out, int k, int n, void* stream);
/* Fused gate/up projection + SwiGLU: w_gu is int8 [2n][k] with rows interleaved (row 2i = gate_i, row 2i+1 = up_i),
 * w_s_gu the matching 2n scales; y[i] = up_i * (gate_i/(1+exp(-gate_i))), gate_i/up_i dequantised as above.
 * = two GEMVs + dec_Swish (Modules/Swish.h:26-41) + dec_Gate_Layer_fp32xfp32 (Modules/Linear_Layer.h:1103-1121). */
int flexllm_linear_i8_gemv_swiglu(const int8_t* x, const float* s_x, const int8_t* w_gu, const float* w_s_gu, float* y,
                                  int k, int n, void* stream);
/* Prefill GEMM, exact: acc[m][n] = sum_k a[m][k]*W[n][k] on int8 MFMA tiles.  Replaces
 * pref_Linear_Layer_i4xi4 (Modules/Linear_Layer.h:293-341) with the int8 systolic array
 * (Modules/MHA.h:113-187, Modules/PE.h:526-583).  k % 64 == 0. */
int flexllm_linear_i8_gemm(const int8_t* a, const int8_t* w, int32_t* acc, int m, int k, int n, void* stream);
/* The same exact product with UNSIGNED 8-bit activations (0..255), the reference's is_uint_input instantiation of its
 * int8 arrays (Modules/MHA.h:339-344, :854-859 with is_uint_input = true; Modules/PE.h:526-583, is_uint_A): used for
 * P.V with the uint8 softmax probabilities as a stand-alone stage.  a [m][k] uint8, w [n][k] int8, acc [m][n] int32;
 * k % 16 == 0; m = 1 is the decode form.  A plain kernel (one wave per output): the fused attention entry points are
 * the fast path. */
int flexllm_linear_u8i8_gemm(const uint8_t* a, const int8_t* w, int32_t* acc, int m, int k, int n, void* stream);
/* Fused prefill linear: y[m][n] = (float(acc)*s_x[m])*w_s[n] (+ residual[m][n]).
 * = GEMM + pref_dequant_layer_qint_fp32 (Modules/quant.h:115-164) (+ pref_Residual_Layer). */
int flexllm_linear_i8_gemm_dequant(const int8_t* a, const float* s_x, const int8_t* w, const float* w_s,
                                   const float* residual, float* y, int m, int k, int n, void* stream);
/* Fused prefill gate/up projection + SwiGLU, the GEMM counterpart of flexllm_linear_i8_gemv_swiglu: w_gu is int8
 * [2n][k] with rows interleaved (row 2i = gate_i, row 2i+1 = up_i), w_s_gu the matching 2n scales;
 * h[m][i] = up_i * (gate_i/(1+exp(-gate_i))) with gate/up = (float(acc)*s_x[m])*w_s_gu[.].  Row m of h equals
 * the GEMV entry point's result for token m bit for bit.  = two pref_Linear_Layer + pref_dequant
 * (Modules/quant.h:115-164) + pref_Swish (Modules/Swish.h:7-24) + pref_Gate_Layer_fp32xfp32
 * (Modules/Linear_Layer.h:1083-1101).  k % 64 == 0, n even. */
int flexllm_linear_i8_gemm_swiglu(const int8_t* a, const float* s_x, const int8_t* w_gu, const float* w_s_gu, float* h,
                                  int m, int k, int n, void* stream);

/* ---- W4A4 linear layers (the reference's shipped configuration) ------------------------------ */
/* Activations asymmetric uint4 (flexllm_quant_asym_u8 with bits=4: value 0..15, scale s_x, zero point b_x = row
 * minimum), weights symmetric int4 (-8..7), both packed two per byte along K: byte j of a row holds element 2j in
 * its low nibble, element 2j+1 in its high nibble (the reference packs two output channels per byte in a
 * port-specific order, SpinQuant_Llama_32_1B/Linear_Layer_Decoding_tb.cpp:176-186; the host adapter repacks).
 * y[n] = (float(acc[n]) * s_x) * w_s[n] + b_x * w_sum[n] (+ residual[n]) with acc = sum_k a[k]*w[n][k] and
 * w_sum[n] = sum_k w[n][k]*w_s[n] supplied by the caller, as the testbench computes it (…_tb.cpp:187-190).
 * Replaces pref_/dec_Linear_Layer_i4xi4 (Modules/Linear_Layer.h:293-341, 862-923) + the asymmetric dequant
 * (Modules/quant.h:146-149). */
/* Packs values held one per byte (low 4 bits used) two per byte; n_values even. */
int flexllm_pack_nibbles(const uint8_t* values, uint8_t* packed, size_t n_values, void* stream);
/* Decode: x4 [k/2], w4 [n][k/2]; k % 32 == 0, k <= 16384. */
int flexllm_linear_u4i4_gemv(const uint8_t* x4, const uint8_t* w4, int32_t* acc, int k, int n, void* stream);
int flexllm_linear_u4i4_gemv_dequant(const uint8_t* x4, const float* s_x, const float* b_x, const uint8_t* w4,
                                     const float* w_s, const float* w_sum, const float* residual, float* y, int k, int n,
                                     void* stream);
/* Prefill: a4 [m][k/2], s_x/b_x [m], w4 [n][k/2]; k % 64 == 0. */
int flexllm_linear_u4i4_gemm(const uint8_t* a4, const uint8_t* w4, int32_t* acc, int m, int k, int n, void* stream);
int flexllm_linear_u4i4_gemm_dequant(const uint8_t* a4, const float* s_x, const float* b_x, const uint8_t* w4,
                                     const float* w_s, const float* w_sum, const float* residual, float* y, int m, int k,
                                     int n, void* stream);
/* The same product on operands held one value per byte: a [m][k] with the unsigned activation values (0..127, e.g.
 * the uint4 output of flexllm_quant_asym_u8 before packing) in int8 containers, w [n][k] int8 (e.g. int4 weights
 * widened once at load time).  Same integer sums and the same dequantisation as flexllm_linear_u4i4_gemm_dequant, on
 * the direct-load MFMA kernel of the int8 path (twice the operand bytes, about half the time at M = 1024).
 * k % 64 == 0, n % 4 == 0.  Replaces pref_Linear_Layer_i4xi4 + the asymmetric dequant like the entry point above. */
int flexllm_linear_i8_gemm_dequant_asym(const int8_t* a, const float* s_x, const float* b_x, const int8_t* w, const float* w_s,
                                        const float* w_sum, const float* residual, float* y, int m, int k, int n, void* stream);
/* The gate/up projection of the same precision with SiLU(gate) * up in the epilogue: w_gu [2n][k] with gate row i at
 * 2i and up row i at 2i+1 (w_s_gu, w_sum_gu [2n] likewise), h [m][n] = up * SiLU(gate) of the dequantised pair - the
 * values flexllm_linear_i8_gemm_dequant_asym followed by flexllm_swiglu_f32 give, bit for bit, with half the output
 * traffic.  Replaces pref_Linear_Layer_i4xi4 (gate, up) + dequant + pref_Swish + pref_Gate_Layer
 * (pref_Swish_Layer_ffn, pref_Gate_Layer_ffn: SpinQuant_Prefilling.h:649-670).  k % 64 == 0. */
int flexllm_linear_i8_gemm_swiglu_asym(const int8_t* a, const float* s_x, const float* b_x, const int8_t* w_gu, const float* w_s_gu,
                                       const float* w_sum_gu, float* h, int m, int k, int n, void* stream);

/* ---- FHT.h ---------------------------------------------------------------------------- */
/* y = H_n x / scale (Sylvester order, butterfly stage order of the reference's omega network, so
 * the fp32 result is bit-identical).  Replaces pref_FHT (Modules/FHT.h:7-67) and dec_FHT
 * (Modules/FHT.h:69-129).  n is a power of two, 1024 <= n <= 8192. In-place allowed. */
int flexllm_fht_f32(const float* x, float* y, int rows, int n, float scale, void* stream);
/* FHT followed by flexllm_quant_sym_i8 on each transformed row, without the fp32 round trip. */
int flexllm_fht_quant_i8(const float* x, int8_t* q, float* s, int rows, int n, float scale, void* stream);
/* FHT followed by flexllm_quant_asym_u8 on each transformed row (the W4A4 graph's input of the down projection,
 * pref_FHT_R4 + pref_quant_layer_ffn_down_fp32_int4, SpinQuant_Prefilling.h:673-700), without the fp32 round trip:
 * the same bytes, scales and minima, bit for bit. */
int flexllm_fht_quant_asym_u8(const float* x, uint8_t* q, float* s, float* b, int bits, int rows, int n, float scale, void* stream);

/* ---- LayerNorm.h ---------------------------------------------------------------------- */
/* RMSNorm: y = (x * (1/sqrt(mean(x^2)+eps))) * gamma.  Replaces pref_Layer_Norm
 * (Modules/LayerNorm.h:28-183) and dec_Layer_Norm (Modules/LayerNorm.h:210-370), beta disabled. */
int flexllm_rmsnorm_f32(const float* x, const float* gamma, float* y, int rows, int dim, float eps, void* stream);
/* RMSNorm followed by flexllm_quant_sym_i8 on each row. */
int flexllm_rmsnorm_quant_i8(const float* x, const float* gamma, int8_t* q, float* s, int rows, int dim,
                             float eps, void* stream);
/* RMSNorm followed by flexllm_quant_asym_u8 on each row (pref_Layer_Norm + pref_quant_layer_fp32_qint<4,true>,
 * SpinQuant_Prefilling.h:78-90, 123-136), one wave per row; dim == 2048.  The sum of squares is taken in the order of the
 * model graphs (512 partial sums of four squares, wave butterflies, eight wave sums in order). */
int flexllm_rmsnorm_quant_asym_u8(const float* x, const float* gamma, uint8_t* q, float* s, float* b, int bits, int rows, int dim,
                                  float eps, void* stream);

/* ---- RoPE.h --------------------------------------------------------------------------- */
/* Rotate-half RoPE from tables sin_t/cos_t [max_pos][head_dim/2]; x,y [tokens][heads][head_dim];
 * token t sits at position pos0+t.  Replaces pref_RoPE_layer (Modules/RoPE.h:8-94) and
 * dec_RoPE_layer (Modules/RoPE.h:96-173). */
int flexllm_rope_f32(const float* x, float* y, const float* sin_t, const float* cos_t, int tokens, int heads,
                     int head_dim, int pos0, void* stream);
/* Host-side table builder (Llama-3 frequency scaling, formula kept in Modules/RoPE.h:28-50);
 * sin_t/cos_t are HOST pointers [max_pos][head_dim/2]. */
int flexllm_rope_table_host(float* sin_t, float* cos_t, int max_pos, int head_dim, float theta, int factor,
                            int low_freq_factor, int high_freq_factor, int original_max_pe);

/* ---- Swish.h / gate / Residual_Layer.h --------------------------------------------------- */
/* y = x/(1+exp(-x)).  pref_Swish / dec_Swish (Modules/Swish.h:5-41). */
int flexllm_swish_f32(const float* x, float* y, size_t n, void* stream);
/* y = up * (gate/(1+exp(-gate))).  Swish + pref/dec_Gate_Layer_fp32xfp32
 * (Modules/Linear_Layer.h:612-630, :1103-1121). */
int flexllm_swiglu_f32(const float* gate, const float* up, float* y, size_t n, void* stream);
/* y = a + b.  pref/dec_Residual_Layer (Modules/Residual_Layer.h:47-87). */
int flexllm_residual_add_f32(const float* a, const float* b, float* y, size_t n, void* stream);

/* ---- Softmax.h / MHA.h --------------------------------------------------------------- */
/* Row softmax with max subtraction.  pref_Softmax (Modules/Softmax.h:6-163), dec_MHA_Softmax
 * (Modules/Softmax.h:456-635). */
int flexllm_softmax_f32(const float* x, float* y, int rows, int dim, void* stream);

/* Static per-head attention scales of one layer (device pointers): Q_s[q_heads], K_s[kv_heads],
 * V_s[kv_heads], A_s[q_heads] (parameters/{Q,K,V,A}_s.h rows, SpinQuant_Llama_32_1B/MHA_i8xi8.h:11-14). */
typedef struct {
    const float* q_s;
    const float* k_s;
    const float* v_s;
    const float* a_s;
} flexllm_mha_scales;

/* int8 KV cache of one layer, head-major so that one head's keys are contiguous:
 *   K: [kv_heads][max_pos][64]              V: [kv_heads][max_pos/64][64 channels][64 positions]
 * (max_pos % 64 == 0).  The reference's 16/32-token line layouts (Modules/MHA.h:74-109, :299-336,
 * :447-515, :741-804) are converted by the host adapter. */
/* Append: quantise k (post-RoPE) and v fp32 [tokens][kv_heads][head_dim] with K_s / V_s and store at
 * positions pos0.. ; replaces the static quant + dec_K/V_cache_buffer/manager write path. */
int flexllm_kv_append_i8(const float* k, const float* v, int8_t* k_cache, int8_t* v_cache,
                         const flexllm_mha_scales* sc, int tokens, int kv_heads, int head_dim, int max_pos,
                         int pos0, void* stream);
/* Fused prefill q/k/v projection: one GEMM over w_qkv int8 [(q_heads + 2 kv_heads)*64][k] = [Wq | Wk | Wv] rows with
 * everything between the projection and attention in its epilogue: dequant, RoPE on q and k (token i at position
 * pos0+i), static int8 quantisation (q by 8*Q_s[h], k by K_s[h], v by V_s[h]) and the stores into q8
 * [m][q_heads][64], the K cache and the transposed V cache blocks.  Bit-identical to
 * flexllm_linear_i8_gemm_dequant -> flexllm_rope_f32 -> flexllm_static_quant_i8 / flexllm_kv_append_i8.
 * = pref_Linear_Layer x3 + pref_dequant (Modules/quant.h:115-164) + pref_RoPE_layer (Modules/RoPE.h:8-94) +
 * pref_static_sym_per_tensor_quant_layer_fp32_qint (Modules/quant.h:252-293) + the K/V cache writers
 * (Modules/MHA.h:74-109, :299-336).  head_dim 64, k % 64 == 0, m % 32 == 0, pos0 % 64 == 0. */
int flexllm_linear_i8_gemm_qkv_rope_cache(const int8_t* a, const float* s_x, const int8_t* w_qkv, const float* w_s,
                                          const float* sin_t, const float* cos_t, const flexllm_mha_scales* sc,
                                          int8_t* q8, int8_t* k_cache, int8_t* v_cache, int m, int k, int q_heads,
                                          int kv_heads, int max_pos, int pos0, void* stream);
/* Same for already-quantised int8 k8/v8 [tokens][kv_heads][head_dim] (pure relayout). */
int flexllm_kv_store_i8(const int8_t* k8, const int8_t* v8, int8_t* k_cache, int8_t* v_cache, int tokens,
                        int kv_heads, int head_dim, int max_pos, int pos0, void* stream);
/* Decode attention for one query token against `len` cached positions (new token already appended):
 * scores=q8.K8 (int32) -> *Q_s*K_s -> softmax -> P=min(255,round(p/A_s)) (uint8) -> P.V8 (int32) -> *A_s*V_s.
 * Replaces the dec_MHA_i8xi8_qxk / dec_MHA_Softmax / quant / dec_MHA_i8xi8_axv chain of
 * SpinQuant_Llama_32_1B/MHA_i8xi8.h:1027-1114.  q8 [q_heads][head_dim]; o fp32 [q_heads][head_dim];
 * p8_out (optional, may be NULL) uint8 [q_heads][len].  head_dim == 64, len <= 8192, q_heads/kv_heads <= 4.
 * Uses a library-owned scratch buffer (allocated on first use, grown with a device synchronisation). */
int flexllm_mha_i8_decode(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache,
                          const flexllm_mha_scales* sc, float* o, uint8_t* p8_out, int len, int q_heads,
                          int kv_heads, int head_dim, int max_pos, void* stream);
/* flexllm_mha_i8_decode for callers that cannot allocate device memory (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc): same arguments, same kernels and bit-identical results, but the scratch (scores,
 * chunk statistics, accumulators: 1 072 KiB) is a fixed array inside the loaded library, one copy per GPU, and the call
 * makes no hipMalloc / hipFree.  It has no counterpart in the reference.  Limits: q_heads <= 32, len <= 8192; larger
 * sizes are rejected with FLEXLLM_EINVAL.  All calls on one GPU share that GPU's array: calls that may overlap on one
 * GPU (different streams) race and must be serialised by the caller.  The first call on a device looks up the array's
 * address (no allocation); make it outside a graph capture. */
int flexllm_mha_i8_decode_noalloc(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache,
                                  const flexllm_mha_scales* sc, float* o, uint8_t* p8_out, int len, int q_heads,
                                  int kv_heads, int head_dim, int max_pos, void* stream);
/* Prefill causal attention over s tokens (positions 0..s-1): q8 [s][q_heads][64] int8; K and V are read from
 * the cache layouts above (filled by flexllm_kv_append_i8 / flexllm_kv_store_i8); o fp32 [s][q_heads][64].
 * Replaces SpinQuant_Llama_32_1B/MHA_i8xi8.h:369-427 from the qxk stage on (pref_MHA_i8xi8_qxk_template,
 * pref_causal_mask_template, pref_Softmax, uint8 P quant, pref_MHA_i8xi8_axv_template, dequant).
 * s % 32 == 0.  p8_out optional uint8 [q_heads][s][s], zero-filled by the caller (only the causal tiles are
 * written). */
int flexllm_mha_i8_prefill(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache,
                           const flexllm_mha_scales* sc, float* o, uint8_t* p8_out, int s, int q_heads,
                           int kv_heads, int head_dim, int max_pos, void* stream);

/* ---- attention with dynamic per-(token, head) scales ---------------------------------------------------------
 * Q, K and V quantised by flexllm_head_quant_sym_i8 (dec_MHA_quant_layer_fp32_qint<8,false>, Modules/quant.h:527-617):
 * one scale per token and head.  Scores are dequantised per key, a[i][j] = (float(q8_i.k8_j) * Q_s[i][h]) * K_s[j][kvh]
 * (the per-token scale streams of Modules/quant.h:165-246 and the K scale cache of Modules/MHA.h:9-71, :393-445) with
 * Q_s = q_s / q_scale_div (sqrt(head_dim) = 8: the factor the static path folds into Q's scale).  V's per-token scale
 * is folded into the probabilities before they are quantised with the same symmetric quantiser:
 * p'[j] = softmax(a)[j] * V_s[j][kvh], s_p = max_j p'[j] / 127, P8 = round(p'/s_p) (int8, 0..127),
 * o[d] = float(sum_j P8[j]*v8[j][d]) * s_p, times v_ch_s[kvh][d] when the reference library's per-channel V scale
 * (Modules/MHA.h:713-738) is given.  K and V are read from the cache layouts of flexllm_kv_store_i8.
 * PARITY: the q.K side (per-token scale streams) has a reference counterpart; the P.V side does not - the reference
 * keeps V's scale static per channel and has no per-token V path, so folding V_s into the probabilities and the int8
 * probabilities 0..127 are this library's own formulation: parity of that stage and of the output is unpinned by the
 * reference (the CPU checker restates the same formulation; it is pinned against a float64 fake-quant golden only). */
typedef struct {
    const float* q_s;      /* prefill: [s][q_heads]; decode: [q_heads]: the quantiser's scales of q */
    const float* k_s;      /* [max_pos][kv_heads]: K scale cache, one scale per position and KV head */
    const float* v_s;      /* [max_pos][kv_heads]: V scale cache */
    const float* v_ch_s;   /* optional [kv_heads][64] per-channel factor on the output, or NULL */
    float q_scale_div;     /* 8.0f for head_dim 64 */
} flexllm_mha_dyn_scales;
/* Causal prefill over s tokens (positions 0..s-1); q8 [s][q_heads][64]; o fp32 [s][q_heads][64]; optional outputs
 * p8_out int8 [q_heads][s][s] (zero-filled by the caller) and p_s_out fp32 [s][q_heads].  s % 32 == 0. */
int flexllm_mha_i8_prefill_dyn(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache,
                               const flexllm_mha_dyn_scales* sc, float* o, int8_t* p8_out, float* p_s_out, int s,
                               int q_heads, int kv_heads, int head_dim, int max_pos, void* stream);
/* One query token against len cached positions; q8 [q_heads][64]; optional p8_out int8 [q_heads][len], p_s_out
 * [q_heads].  len <= 8192, q_heads/kv_heads <= 4.  Uses a library-owned scratch buffer like flexllm_mha_i8_decode. */
int flexllm_mha_i8_decode_dyn(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache,
                              const flexllm_mha_dyn_scales* sc, float* o, int8_t* p8_out, float* p_s_out, int len,
                              int q_heads, int kv_heads, int head_dim, int max_pos, void* stream);

/* ---- Logits.h (greedy and top-k sampling) ---------------------------------------------- */
/* logits[v] = sum_k fp16(E[v][k]) * n[k] (fp32 accumulate): tied fp16 lm_head GEMV. */
int flexllm_lm_head_f16(const uint16_t* embed, const float* n, float* logits, int vocab, int hidden, void* stream);
/* Index of the maximum (lowest index on ties); result is a device int. */
int flexllm_argmax_f32(const float* x, int n, int* result, void* stream);
/* Top-k sampling of the next token: the k largest logits, softmax over them (exp(v_k - v_0) when enable_sub_max,
 * two partial sums), cumulative distribution, the first k with rand < cdf[k] (the last candidate otherwise).
 * Replaces the selection/sampling part of dec_Sampling_Embedding_Layer (Modules/Logits.h:145-279, insertion
 * routine :5-31); the embedding look-up that follows there is flexllm_embed_f16.  rand: device pointer to one
 * float in [0,1) (the reference's host-supplied rand_seed); token: device int.  top_idx/top_val/top_prob
 * (optional, device, [top_k]) return the candidates in rank order.  Equal logits are ranked by index (the
 * reference ranks them by its lane scan order; values and probabilities are the same).  1 <= top_k <= 16. */
int flexllm_sample_topk_f32(const float* logits, int n, int top_k, const float* rand, int enable_sub_max, int* token,
                            int* top_idx, float* top_val, float* top_prob, void* stream);
/* y = fp32(E[token]) with the token id read from device memory.  The table's row count is not known here: the
 * caller guarantees 0 <= token < rows (the model entry points below check ids against their vocabulary). */
int flexllm_embed_f16(const uint16_t* embed, const int* token, float* y, int hidden, void* stream);

/* ---- whole model: Llama-3.2-1B W8A8 SpinQuant graph ------------------------------------- */
/* Layer order of SpinQuant_Llama_32_1B/SpinQuant_Prefilling.h:940-1049 and
 * SpinQuant_Decoding_mem_opt.h:1050-1126 with int8 symmetric linear layers. */
typedef struct {
    int layers, hidden, kv_hidden, inter, q_heads, kv_heads, head_dim, vocab, max_pos;
    float eps, fht_scale;
} flexllm_llama_config;

typedef struct {
    /* arrays of `layers` device pointers (host arrays of device pointers) */
    const int8_t* const* wq; const int8_t* const* wk; const int8_t* const* wv; const int8_t* const* wo;
    const int8_t* const* wg; const int8_t* const* wu; const int8_t* const* wd;
    const float* const* sq; const float* const* sk; const float* const* sv; const float* const* so;
    const float* const* sg; const float* const* su; const float* const* sd;
    const float* gamma;                 /* device [2*layers+1][hidden] */
    const float* q_s; const float* k_s; const float* v_s; const float* a_s; /* device [layers][heads] */
    const float* rope_sin; const float* rope_cos;                           /* device [max_pos][head_dim/2] */
    const uint16_t* embed;              /* device fp16 [vocab][hidden] */
} flexllm_llama_weights;

typedef struct flexllm_llama flexllm_llama;

/* Copies/repacks the weights into the library's own device layout (fused qkv and gate/up rows) and
 * allocates the int8 KV caches (per layer in the head-major layouts given above for flexllm_kv_append_i8:
 * K [layers][kv_heads][max_pos][64], V [layers][kv_heads][max_pos/64][64 channels][64 positions]) and the
 * activation workspace. */
int flexllm_llama_create(flexllm_llama** out, const flexllm_llama_config* cfg, const flexllm_llama_weights* w);
/* The shipped W4A4 configuration as a model of its own: asymmetric uint4 activations x int4 weights in all seven
 * projections and in the output head (one int4 engine for every linear layer and an int4 lm_head in
 * SpinQuant_Llama_32_1B/SpinQuant_Decoding_mem_opt.h:363-365, 415-469), int8 attention as above.  `base` holds the
 * matrices as int8 arrays of int4 values (-8..7, one per byte, as in parameters/<proj>_L%02d.bin) with their scales,
 * and the fp16 embedding table that turns a token id into the layer input; sum<p>[l] is the per-output-row sum of
 * the dequantised weights (the generated headers' w_<proj>_sum), which the activations' zero point multiplies; the
 * head is int4 [vocab][hidden] one value per byte with per-row scale and row sum.  The library packs the matrices two
 * values per byte for the decode kernel and keeps the byte-held copy for the prefill GEMMs (1.5 x the packed weight
 * memory); a value outside -8..7 anywhere in the matrices or the head is refused with FLEXLLM_EINVAL, because the two
 * copies would otherwise disagree (the packed one keeps the low nibble).  Decoding (flexllm_llama_decode_hidden / _decode_greedy / _decode_sample) runs in the persistent
 * kernel only, which then streams half the weight bytes per token.  flexllm_llama_prefill_hidden and
 * flexllm_llama_generate run the configuration's prefill graph (SpinQuant_Prefilling.h:807-1050): per-token asymmetric
 * uint4 quantisation, the 4-bit values multiplied one per byte on the int8 MFMA kernel with zero point x row sum in its
 * epilogue, RoPE + static quantisation + cache stores, int8 attention, SiLU(gate)*up and the Hadamard transform. */
typedef struct {
    flexllm_llama_weights base;
    const float* const* sumq; const float* const* sumk; const float* const* sumv; const float* const* sumo;
    const float* const* sumg; const float* const* sumu; const float* const* sumd;
    const int8_t* head_w;               /* device int4 values [vocab][hidden], one per byte */
    const float* head_s;                /* device [vocab] */
    const float* head_sum;              /* device [vocab] */
} flexllm_llama_w4a4_weights;
int flexllm_llama_create_w4a4(flexllm_llama** out, const flexllm_llama_config* cfg, const flexllm_llama_w4a4_weights* w);
int flexllm_llama_destroy(flexllm_llama* m);
/* Decode schedule: 0 (default) = one persistent kernel per token (all layers + lm_head, grid barriers between
 * stages, next stage's weights prefetched across the barrier) when the device has >= 256 CUs and the shapes are
 * Llama-3.2-1B's with max_pos <= 4096; 1 = one kernel per stage.  Same arithmetic either way. */
int flexllm_llama_set_decode_mode(flexllm_llama* m, int mode);
/* Debug aid: the first call switches stage stamping on; later calls copy out workgroup 0's 100 MHz wall-clock
 * stamps of the last persistent decode step: per layer 6 x (stage start after the barrier, stage end before the
 * next arrive), then the head's start and end. */
int flexllm_llama_stage_timeline(flexllm_llama* m, long long* host_out, int max_entries);
/* How the persistent decode kernel's exchange memory was placed when the model was created (no counterpart in the
 * reference).  The GPU is two I/O dies with four XCDs and half of the HBM each; a word handed from one workgroup to
 * another through memory of the other die takes longer, and memory alternates between the dies in 8 KiB blocks.
 * flexllm_llama_create measures which die each block of a small arena belongs to (about 10 ms) and keeps every
 * exchanged array once per die: producers store into both copies, consumers poll their own die's.
 *   *two_copies  1 when the measurement succeeded; 0 when the arrays exist once (fewer than 256 CUs, workgroups not
 *                dealt round-robin to eight XCDs, no clear difference between the blocks, or FLEXLLM_DIE_COPIES=0
 *                in the environment when the model was created).  Results are the same either way.
 *   *die_mask    bit x = the die of XCD x
 *   *near_us, *far_us   mean time of one exchange round among the 32 workgroups of an XCD through memory of their
 *                own die / of the other die, as measured (0 when two_copies is 0) */
int flexllm_llama_exchange_info(const flexllm_llama* m, int* two_copies, unsigned* die_mask, float* near_us, float* far_us);
/* The arithmetic of that measurement, on the host alone (no GPU needed; exported so that it can be checked on made-up
 * timings).  us[b * 8 + x] = exchange round of XCD x's workgroups through block b, microseconds.  XCDs whose timings
 * correlate with XCD 0's over the blocks are die 0 (*die_mask: bit x = die of XCD x); die_of_block[b] = the die whose
 * four XCDs are at least 4 % faster through block b, or -1.  *usable = 0 - and the library would keep one copy - unless
 * each die has four XCDs and at least four blocks; *near_us / *far_us = mean round through own-die / other-die blocks. */
int flexllm_die_classify(const float* us, int n_blocks, int* usable, unsigned* die_mask, int* die_of_block, float* near_us, float* far_us);
/* Synchronises the device and reports what a decode run flagged on the device: a grid barrier of the persistent
 * kernel that timed out (FLEXLLM_EHIP), or an input token id outside the vocabulary (FLEXLLM_EINVAL; token 0 was
 * used in its place, no row outside the embedding table is ever read).  Clears the flag. */
int flexllm_llama_check(flexllm_llama* m);
/* Device pointers to the int8 caches for inspection / pre-filling.  They are NOT token-major: layer l starts at byte
 * l * kv_heads * max_pos * 64 of each, K as [kv_heads][max_pos][64], V as [kv_heads][max_pos/64][64 channels]
 * [64 positions].  flexllm_kv_store_i8 writes token-major int8 rows [tokens][kv_heads][64] into one layer's pair. */
int flexllm_llama_kv_cache(flexllm_llama* m, int8_t** k_cache, int8_t** v_cache);
/* One decode step at position pos from fp32 embedding x_in (device, [hidden]); writes the residual
 * stream after the last layer to hidden_out (device, may be NULL) and, if logits != NULL, the fp32
 * logits [vocab]. */
int flexllm_llama_decode_hidden(flexllm_llama* m, const float* x_in, int pos, float* hidden_out, float* logits,
                                void* stream);
/* Greedy generation loop on the device: starting from token id *token_io (device int) at position pos0,
 * runs `steps` decode steps (embedding lookup -> 16 layers -> final norm -> lm_head -> argmax), writes the
 * generated ids to tokens_out (device int[steps]).  With use_graph != 0 one step is captured in a HIP graph
 * and replayed. */
int flexllm_llama_decode_greedy(flexllm_llama* m, int* token_io, int pos0, int steps, int* tokens_out,
                                int use_graph, void* stream);
/* Generation with top-k sampling, the reference's own loop (SpinQuant_Decoding_mem_opt.h:924-940 with
 * dec_Sampling_Embedding_Layer, Modules/Logits.h:145-279; host random numbers as in
 * SpinQuant_Prefilling_Decoding_mem_opt_tb.cpp:827-830): for step s the token is drawn from the top_k logits
 * with rands[s] (device array of `steps` floats in [0,1)), written to tokens_out[s] (device) and fed back through
 * token_io (device int, holds the first input token on entry).  On the persistent-kernel schedule the selection and
 * the draw happen inside the kernel, up to 64 tokens per launch. */
int flexllm_llama_decode_sample(flexllm_llama* m, int* token_io, int pos0, int steps, const float* rands, int top_k,
                                int* tokens_out, void* stream);
/* Prompt to tokens, the flow of the reference's combined harness (SpinQuant_Prefilling_Decoding_mem_opt_tb.cpp:753-930):
 * all prompt tokens but the last are embedded and prefilled (positions 0..n_prompt-2; the rows are padded to the
 * prefill tile with zero rows, whose cache entries the decode steps overwrite before they are read), the last prompt
 * token is the first input of the decode loop at position n_prompt-1, and `steps` tokens are generated into
 * tokens_out (device): greedy when top_k == 0, else top-k sampling with rands[step] (device, `steps` floats in [0,1)).
 * prompt: device int [n_prompt], n_prompt >= 1, n_prompt - 1 + steps <= max_pos.  Token ids outside the vocabulary are
 * reported by flexllm_llama_check. */
int flexllm_llama_generate(flexllm_llama* m, const int* prompt, int n_prompt, int steps, const float* rands, int top_k,
                           int* tokens_out, void* stream);
/* Prefill s tokens at positions 0..s-1 from fp32 embeddings x_in (device [s][hidden]); fills the KV cache,
 * writes the residual stream to hidden_out (device [s][hidden], may be NULL). */
int flexllm_llama_prefill_hidden(flexllm_llama* m, const float* x_in, int s, float* hidden_out, void* stream);

/* ---- HMT long-context plug-in (Modules/HMT.h, HMT_SpinQuant_Llama_32_1B/HMT_SpinQuant_Unit.h) ----------------
 * The plug-in runs the layer stack (flexllm_llama_prefill_hidden) twice per segment on assembled sequences and
 * keeps a ring of memory embeddings; these entry points are its fp32 pieces.  All pointers are device pointers. */
/* y[n] = sum_k w[n][k] * x[k] in fp32 (w row-major [n][k], k % 4 == 0).  dec_Linear_Layer_fp32xfp32
 * (Modules/Linear_Layer.h:1041-1100), used for the query Q_n = Wq S_n and the key K_n = Wk M_n
 * (Modules/HMT.h:289-292, :306-311). */
int flexllm_linear_f32_gemv(const float* x, const float* w, float* y, int k, int n, void* stream);
/* Memory retrieval: a[j] = q . kmem[j] over ALL mem_num slots (empty slots are zero rows and take part),
 * a_sft = softmax((a - max) / scale), p_out[c] = sum_j a_sft[j] * mmem[j][c].  kmem, mmem: [mem_num][hidden].
 * hmt_Linear_Layer_fp32xfp32_qk_attn_template (Modules/HMT.h:278-316) + hmt_attn_softmax with enable_scale,
 * enable_sub_max (HMT_SpinQuant_Unit.h:96-105; Modules/Softmax.h:262-360).  mem_num <= 1024. */
int flexllm_hmt_retrieve(const float* q, const float* kmem, const float* mmem, float* a_sft, float* p_out, int mem_num,
                         int hidden, float scale, void* stream);
/* Input sequence of one stage of hmt_segment_loader_sync_template (Modules/HMT.h:48-98 stage 0, :125-170 stage 1),
 * written to x_out [rows][hidden], rows beyond the sequence zero:
 *   stage 0: [t_embed, emb[seq_off .. seq_off+cur_sum_len), t_embed]
 *   stage 1: [p_buf, emb[seq_off-rec_len .. seq_off) (zero rows before the text), emb[seq_off .. seq_off+cur_len),
 *             p_buf if tail_p]
 * emb: [seq_len][hidden] token embeddings. */
int flexllm_hmt_stage_input(const float* emb, const float* t_embed, const float* p_buf, float* x_out, int stage, int seq_off,
                            int cur_len, int cur_sum_len, int rec_len, int tail_p, int rows, int hidden, void* stream);

#ifdef __cplusplus
}
#endif
#endif

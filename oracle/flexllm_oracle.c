/*
 * CPU oracle for the FlexLLM quantized-transformer datapath: TEST INFRASTRUCTURE ONLY
 * (see flexllm_oracle.h).  Build: gcc -O2 -ffp-contract=off -fno-fast-math -shared -fPIC.
 */
#include "flexllm_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* The loops over independent outputs (rows of a matrix product, heads and query rows of attention, vocabulary rows)
 * are OpenMP loops: every output is computed by one thread with the same scalar code, so the results do not depend on
 * the thread count.  fxo_set_threads(1) gives the single-core baseline. */
void fxo_set_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n > 0 ? n : omp_get_num_procs());
#else
    (void)n;
#endif
}
int fxo_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ quant.h */

static void row_min_max(const float* x, int dim, float* mx, float* mn) {
    /* Modules/quant.h:24-43: running max/min from +-1e32 with strict compares. */
    float vmax = (float)-1e32, vmin = (float)1e32;
    for (int k = 0; k < dim; k++) {
        if (x[k] > vmax) vmax = x[k];
        if (x[k] < vmin) vmin = x[k];
    }
    *mx = vmax; *mn = vmin;
}

void fxo_quant_sym(const float* x, int rows, int dim, int bits, int8_t* q, float* s) {
    const float scale_base = (float)((1 << (bits - 1)) - 1);            /* quant.h:85 */
    for (int r = 0; r < rows; r++) {
        const float* xr = x + (size_t)r * dim;
        float vmax, vmin;
        row_min_max(xr, dim, &vmax, &vmin);
        float amax = fabsf(vmax), amin = fabsf(vmin);                    /* quant.h:89-90 */
        float sc = (amax > amin ? amax : amin) / scale_base;            /* quant.h:91 */
        if (sc == 0) sc = 1;                                             /* quant.h:92 */
        s[r] = sc;
        for (int k = 0; k < dim; k++) {
            float t = xr[k] / sc;                                        /* quant.h:102 */
            q[(size_t)r * dim + k] = (int8_t)(int)roundf(t);             /* quant.h:103 */
        }
    }
}

void fxo_quant_asym(const float* x, int rows, int dim, int bits, uint8_t* q, float* s, float* b) {
    const float scale_base = (float)((1 << bits) - 1);                  /* quant.h:54 */
    for (int r = 0; r < rows; r++) {
        const float* xr = x + (size_t)r * dim;
        float vmax, vmin;
        row_min_max(xr, dim, &vmax, &vmin);
        float sc = (vmax - vmin) / scale_base;                           /* quant.h:61 */
        if (sc == 0) sc = 1;
        s[r] = sc; b[r] = vmin;                                          /* quant.h:63 */
        for (int k = 0; k < dim; k++) {
            float t = (xr[k] - vmin) / sc;                               /* quant.h:75 */
            q[(size_t)r * dim + k] = (uint8_t)((unsigned)(int)roundf(t) & ((1u << bits) - 1u));
        }
    }
}

void fxo_dequant(const int32_t* acc, int rows, int n, const float* s_x, const float* b_x,
                 const float* w_s, const float* w_sum, float* y) {
    for (int r = 0; r < rows; r++)
        for (int j = 0; j < n; j++) {
            float t = (float)acc[(size_t)r * n + j] * s_x[r] * w_s[j];  /* quant.h:147,151 */
            if (b_x && w_sum) t = t + b_x[r] * w_sum[j];                 /* quant.h:148 */
            y[(size_t)r * n + j] = t;
        }
}

void fxo_static_quant(const float* x, int rows, int heads, int dim, const float* scale,
                      float factor, int is_signed, int bits, int8_t* q) {
    const int scale_base = is_signed ? (1 << (bits - 1)) : (1 << bits); /* quant.h:262 */
    for (int r = 0; r < rows; r++)
        for (int h = 0; h < heads; h++)
            for (int k = 0; k < dim; k++) {
                size_t i = ((size_t)r * heads + h) * dim + k;
                float t = x[i] / (factor * scale[h]);                    /* quant.h:272 */
                int rt = (int)roundf(t);                                 /* quant.h:273 */
                int o;
                if (is_signed) o = rt > scale_base - 1 ? scale_base - 1 : rt < -scale_base ? -scale_base : rt;
                else o = rt > scale_base - 1 ? scale_base - 1 : rt;      /* quant.h:275-280 */
                q[i] = (int8_t)(o & 0xff);
            }
}

void fxo_static_dequant(const int32_t* acc, int rows, int act_heads, int w_heads, int dim,
                        const float* a_s, const float* w_s, float* y) {
    const int group = act_heads / w_heads;
    for (int r = 0; r < rows; r++)
        for (int h = 0; h < act_heads; h++)
            for (int k = 0; k < dim; k++) {
                size_t i = ((size_t)r * act_heads + h) * dim + k;
                y[i] = (float)acc[i] * a_s[h] * w_s[h / group];          /* quant.h:315, :793-795 */
            }
}

void fxo_head_quant_sym(const float* x, int rows, int heads, int dim, int bits, int8_t* q, float* s) {
    fxo_quant_sym(x, rows * heads, dim, bits, q, s);                    /* quant.h:591-615: same math per head */
}

/* ------------------------------------------------ Linear_Layer.h (int GEMM) */

void fxo_linear_i8(const int8_t* a, const int8_t* w, int m, int k, int n, int32_t* c) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = 0; i < m; i++)
        for (int j = 0; j < n; j++) {
            const int8_t* ar = a + (size_t)i * k;
            const int8_t* wr = w + (size_t)j * k;
            int32_t acc = 0;
            for (int t = 0; t < k; t++) acc += (int32_t)ar[t] * (int32_t)wr[t];
            c[(size_t)i * n + j] = acc;
        }
}

void fxo_linear_u8i8(const uint8_t* a, const int8_t* w, int m, int k, int n, int32_t* c) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = 0; i < m; i++)
        for (int j = 0; j < n; j++) {
            const uint8_t* ar = a + (size_t)i * k;
            const int8_t* wr = w + (size_t)j * k;
            int32_t acc = 0;
            for (int t = 0; t < k; t++) acc += (int32_t)ar[t] * (int32_t)wr[t];
            c[(size_t)i * n + j] = acc;
        }
}

/* -------------------------------------------------------------------- FHT.h */

void fxo_fht(const float* x, int rows, int n, float scale, float* y) {
    int m = 0;
    while ((1 << m) < n) m++;
    float* buf0 = (float*)malloc(sizeof(float) * n);
    float* buf1 = (float*)malloc(sizeof(float) * n);
    float* shuf = (float*)malloc(sizeof(float) * n);
    for (int r = 0; r < rows; r++) {
        float* cur = buf0; float* nxt = buf1;
        memcpy(cur, x + (size_t)r * n, sizeof(float) * n);
        for (int s = 0; s < m; s++) {
            for (int i = 0; i < n; i++) {                                /* FHT.h:33-38 perfect shuffle */
                int idx = ((i << 1) & (n - 1)) | (i >> (m - 1));
                shuf[i] = cur[idx];
            }
            for (int i = 0; i < n; i += 2) {                             /* FHT.h:40-52 exchange */
                float u = shuf[i], v = shuf[i + 1];
                nxt[i] = u + v;
                nxt[i + 1] = u - v;
            }
            float* t = cur; cur = nxt; nxt = t;
        }
        for (int i = 0; i < n; i++) y[(size_t)r * n + i] = cur[i] / scale; /* FHT.h:58-65 */
    }
    free(buf0); free(buf1); free(shuf);
}

/* -------------------------------------------------------------- LayerNorm.h */

void fxo_rmsnorm_pref(const float* x, const float* gamma, int rows, int dim, float eps, float* y) {
    for (int r = 0; r < rows; r++) {
        const float* xr = x + (size_t)r * dim;
        float p[4] = {0, 0, 0, 0};
        for (int k = 0; k < dim / 4; k++)                                /* LayerNorm.h:82-108 */
            for (int j = 0; j < 4; j++) { float t = xr[4 * k + j]; p[j] += t * t; }
        float rms = 1.0f / sqrtf(((p[0] + p[1]) + (p[2] + p[3])) / (float)dim + eps); /* :112-114 */
        for (int k = 0; k < dim; k++) y[(size_t)r * dim + k] = xr[k] * rms * gamma[k];  /* :121 */
    }
}

void fxo_rmsnorm_dec(const float* x, const float* gamma, int dim, int bp, float eps, float* y) {
    const int per = dim / bp;
    float total = 0;
    float* lane = (float*)malloc(sizeof(float) * bp);
    for (int i = 0; i < bp; i++) {
        float p[4] = {0, 0, 0, 0};
        for (int k = 0; k < per / 4; k++)                                /* LayerNorm.h:263-288 */
            for (int j = 0; j < 4; j++) { float t = x[i * per + 4 * k + j]; p[j] += t * t; }
        lane[i] = (p[0] + p[1]) + (p[2] + p[3]);                         /* :290-294 */
    }
    for (int i = 0; i < bp; i++) total += lane[i];                       /* :296-299 */
    free(lane);
    float rms = 1.0f / sqrtf(total / (float)dim + eps);                 /* :302 */
    for (int k = 0; k < dim; k++) y[k] = x[k] * rms * gamma[k];          /* :308 */
}

/* ------------------------------------------------------------------- RoPE.h */

void fxo_rope_table(int max_pos, int head_dim, float theta, int factor, int low_freq_factor,
                    int high_freq_factor, int original_max_pe, float* sin_t, float* cos_t) {
    const int half = head_dim / 2;
    const int high_wave_length = original_max_pe / high_freq_factor;     /* RoPE.h:28 */
    const int low_wave_length = original_max_pe / low_freq_factor;       /* RoPE.h:29 */
    for (int i = 0; i < half; i++) {
        float exponent = (2.0f * i) / (float)head_dim;                   /* RoPE.h:31 */
        float inv_freq = powf(theta, exponent);                          /* RoPE.h:32 */
        float freq = 1.0f / inv_freq;                                    /* RoPE.h:33 */
        float wavelength = (float)(2 * M_PI * inv_freq);                 /* RoPE.h:34 */
        float scale_freq;
        if (wavelength < high_wave_length) scale_freq = freq;            /* RoPE.h:37-38 */
        else if (wavelength > low_wave_length) scale_freq = freq / factor;
        else {
            float a = (original_max_pe / wavelength - low_freq_factor) / (high_freq_factor - low_freq_factor);
            scale_freq = (1 - a) * (freq / factor) + a * freq;          /* RoPE.h:42-43 */
        }
        for (int s = 0; s < max_pos; s++) {
            float th = s * scale_freq;                                   /* RoPE.h:47 */
            sin_t[(size_t)s * half + i] = sinf(th);
            cos_t[(size_t)s * half + i] = cosf(th);
        }
    }
}

void fxo_rope(const float* x, int tokens, int heads, int head_dim, const float* sin_t,
              const float* cos_t, int pos0, float* y) {
    const int half = head_dim / 2;
    for (int t = 0; t < tokens; t++)
        for (int h = 0; h < heads; h++) {
            const float* xi = x + ((size_t)t * heads + h) * head_dim;
            float* yo = y + ((size_t)t * heads + h) * head_dim;
            const float* sn = sin_t + (size_t)(pos0 + t) * half;
            const float* cs = cos_t + (size_t)(pos0 + t) * half;
            for (int k = 0; k < half; k++) {
                float t0 = xi[k], t1 = xi[k + half];
                yo[k] = t0 * cs[k] - t1 * sn[k];                         /* RoPE.h:77 */
                yo[k + half] = t0 * sn[k] + t1 * cs[k];                  /* RoPE.h:78 */
            }
        }
}

/* -------------------------------------------- Swish.h / gate / Residual_Layer.h */

void fxo_swish(const float* x, int n, float* y) {
    for (int i = 0; i < n; i++) y[i] = x[i] / (1 + expf(-x[i]));          /* Swish.h:19 */
}
void fxo_gate(const float* a, const float* b, int n, float* y) {
    for (int i = 0; i < n; i++) y[i] = a[i] * b[i];                       /* Linear_Layer.h:1116 */
}
void fxo_residual(const float* a, const float* b, int n, float* y) {
    for (int i = 0; i < n; i++) y[i] = a[i] + b[i];                       /* Residual_Layer.h:61 */
}

/* ---------------------------------------------------------------- Softmax.h */

static void softmax_row(const float* x, int dim, float* y) {
    float mx = (float)-1e32;                                              /* Softmax.h:36 */
    for (int k = 0; k < dim; k++) mx = x[k] > mx ? x[k] : mx;             /* Softmax.h:45 */
    float p[4] = {0, 0, 0, 0};
    for (int k = 0; k < (dim + 3) / 4; k++)                               /* Softmax.h:54-94, :516-554 */
        for (int j = 0; j < 4; j++)
            if (4 * k + j < dim) {
                float t = expf(x[4 * k + j] - mx);
                y[4 * k + j] = t;
                p[j] += t;
            }
    float cd = 1.0f / ((p[0] + p[1]) + (p[2] + p[3]));                    /* Softmax.h:145-150 */
    for (int k = 0; k < dim; k++) y[k] = y[k] * cd;                       /* Softmax.h:151-160 */
}

void fxo_softmax(const float* x, int rows, int dim, float* y) {
    for (int r = 0; r < rows; r++) softmax_row(x + (size_t)r * dim, dim, y + (size_t)r * dim);
}

/* dec_Softmax (Softmax.h:262-360), the vector form used outside attention: the dim inputs are block-partitioned over
 * bp lanes (lane i holds elements i*dim/bp ... ), exp((x - max) / scale) when enable_scale (:313), partial sums per
 * lane and per k % 4 (:316), lane sums (p0+p1)+(p2+p3) (:337-342), lanes added in order (:344-347), one reciprocal (:349). */
void fxo_softmax_dec(const float* x, int dim, int bp, int enable_scale, float scale, float* y) {
    float mx = (float)-1e32;                                              /* :287 */
    for (int k = 0; k < dim; k++) mx = x[k] > mx ? x[k] : mx;             /* :297-305 */
    const int per = dim / bp;
    float total = 0.0f;
    for (int i = 0; i < bp; i++) {
        float p[4] = {0, 0, 0, 0};
        for (int k = 0; k < per; k++) {
            const float d = x[i * per + k] - mx;
            const float t = enable_scale ? expf(d / scale) : expf(d);
            y[i * per + k] = t;
            p[k % 4] += t;
        }
        total += (p[0] + p[1]) + (p[2] + p[3]);
    }
    const float cd = 1.0f / total;
    for (int k = 0; k < dim; k++) y[k] = y[k] * cd;                       /* :351-360 */
}

/* dec_Linear_Layer_fp32xfp32 (Linear_Layer.h:1041-1100) on PE_fp32xfp32_pack_1x2_1D (PE.h:709-752): y[n] = sum_k
 * w[n][k] * x[k] in fp32 with four partial sums by k % 4 joined as (p0+p1)+(p2+p3) (tree_adder_4, PE.h:86-90). */
void fxo_linear_f32(const float* x, const float* w, int k, int n, float* y) {
    for (int r = 0; r < n; r++) {
        float p[4] = {0, 0, 0, 0};
        for (int i = 0; i < k; i++) p[i % 4] += x[i] * w[(size_t)r * k + i];
        y[r] = (p[0] + p[1]) + (p[2] + p[3]);
    }
}

/* Memory retrieval of the HMT plug-in (HMT.h:278-316, HMT_SpinQuant_Unit.h:96-105): scores a[j] = q . kmem[j] over ALL
 * mem_num slots (empty slots hold zeros and take part), softmax((a - max) / scale) over the slots, p = sum_j a[j] *
 * mmem[j] computed as a linear layer whose weight row c is column c of the memory matrix. */
void fxo_hmt_retrieve(const float* q, const float* kmem, const float* mmem, int mem_num, int hidden, int bp,
                      float scale, float* a_sft, float* p_out) {
    float a[1024];
    fxo_linear_f32(q, kmem, hidden, mem_num, a);
    fxo_softmax_dec(a, mem_num, bp, 1, scale, a_sft);
    for (int c = 0; c < hidden; c++) {
        float p[4] = {0, 0, 0, 0};
        for (int j = 0; j < mem_num; j++) p[j % 4] += a_sft[j] * mmem[(size_t)j * hidden + c];
        p_out[c] = (p[0] + p[1]) + (p[2] + p[3]);
    }
}

void fxo_causal_mask(const float* x, int rows, int heads, int dim, float* y) {
    for (int r = 0; r < rows; r++)
        for (int h = 0; h < heads; h++)
            for (int k = 0; k < dim; k++) {
                size_t i = ((size_t)r * heads + h) * dim + k;
                y[i] = (k <= r) ? x[i] : (float)-1e32;                    /* MHA.h:262-267 */
            }
}

/* ------------------------------------------------- MHA_i8xi8.h whole attention */

/* The attention proper on already quantised tensors.  p8_in != NULL replaces the probabilities this function would
 * compute (a test feeds the device's own probability bytes back to isolate the P.V stage behind a rounding tie). */
void fxo_mha_prefill_i8(const int8_t* q8, const int8_t* k8, const int8_t* v8, int s, int q_heads, int kv_heads,
                        int hd, const fxo_mha_scales* sc, const uint8_t* p8_in, uint8_t* p8_out, float* o) {
    const int group = q_heads / kv_heads;
#pragma omp parallel
    {
    float* row = (float*)malloc(sizeof(float) * s);
    float* prob = (float*)malloc(sizeof(float) * s);
    uint8_t* p8 = (uint8_t*)malloc((size_t)s);
#pragma omp for collapse(2) schedule(dynamic, 8)
    for (int h = 0; h < q_heads; h++) {
        for (int i = 0; i < s; i++) {
            const int kh = h / group;                                     /* MHA.h:96-106 */
            const int8_t* qi = q8 + ((size_t)i * q_heads + h) * hd;
            if (p8_in) {
                memcpy(p8, p8_in + ((size_t)h * s + i) * s, (size_t)s);
            } else {
                for (int j = 0; j < s; j++) {
                    const int8_t* kj = k8 + ((size_t)j * kv_heads + kh) * hd;
                    int32_t acc = 0;                                      /* MHA.h:189-243 */
                    for (int d = 0; d < hd; d++) acc += (int32_t)qi[d] * (int32_t)kj[d];
                    float a = (float)acc * sc->q_s[h] * sc->k_s[kh];      /* MHA_i8xi8.h:154 -> quant.h:315 */
                    row[j] = (j <= i) ? a : (float)-1e32;                 /* MHA.h:262-267 */
                }
                softmax_row(row, s, prob);                                /* MHA_i8xi8.h:231 */
                for (int j = 0; j < s; j++) {                             /* MHA_i8xi8.h:254: unsigned, base 256 */
                    float t = prob[j] / (1.0f * sc->a_s[h]);
                    int rt = (int)roundf(t);
                    p8[j] = (uint8_t)(rt > 255 ? 255 : rt);
                }
            }
            if (p8_out) memcpy(p8_out + ((size_t)h * s + i) * s, p8, (size_t)s);
            if (o)
                for (int d = 0; d < hd; d++) {
                    int32_t acc = 0;                                      /* MHA.h:339-389, is_uint_input */
                    for (int j = 0; j < s; j++)
                        acc += (int32_t)p8[j] * (int32_t)v8[((size_t)j * kv_heads + kh) * hd + d];
                    o[((size_t)i * q_heads + h) * hd + d] = (float)acc * sc->a_s[h] * sc->v_s[kh]; /* :351 */
                }
        }
    }
    free(row); free(prob); free(p8);
    }
}

void fxo_mha_prefill(const float* q, const float* k, const float* v, int s, int q_heads, int kv_heads,
                     int hd, const fxo_mha_scales* sc, int8_t* q8_out, int8_t* k8_out, int8_t* v8_out,
                     uint8_t* p8_out, float* o) {
    int8_t* q8 = (int8_t*)malloc((size_t)s * q_heads * hd);
    int8_t* k8 = (int8_t*)malloc((size_t)s * kv_heads * hd);
    int8_t* v8 = (int8_t*)malloc((size_t)s * kv_heads * hd);
    /* MHA_i8xi8.h:40-42 (q, with sqrt(head_dim) folded in), :71-73 (k), :285-287 (v) */
    fxo_static_quant(q, s, q_heads, hd, sc->q_s, sqrtf((float)hd), 1, 8, q8);
    fxo_static_quant(k, s, kv_heads, hd, sc->k_s, 1.0f, 1, 8, k8);
    fxo_static_quant(v, s, kv_heads, hd, sc->v_s, 1.0f, 1, 8, v8);
    fxo_mha_prefill_i8(q8, k8, v8, s, q_heads, kv_heads, hd, sc, NULL, p8_out, o);
    if (q8_out) memcpy(q8_out, q8, (size_t)s * q_heads * hd);
    if (k8_out) memcpy(k8_out, k8, (size_t)s * kv_heads * hd);
    if (v8_out) memcpy(v8_out, v8, (size_t)s * kv_heads * hd);
    free(q8); free(k8); free(v8);
}

void fxo_mha_decode(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache, int len,
                    int q_heads, int kv_heads, int hd, const fxo_mha_scales* sc,
                    uint8_t* p8_out, float* o) {
    const int group = q_heads / kv_heads;
#pragma omp parallel
    {
    float* row = (float*)malloc(sizeof(float) * len);
    float* prob = (float*)malloc(sizeof(float) * len);
    uint8_t* p8 = (uint8_t*)malloc((size_t)len);
#pragma omp for schedule(static)
    for (int h = 0; h < q_heads; h++) {
        const int kh = h / group;
        const int8_t* qi = q8 + (size_t)h * hd;
        for (int j = 0; j < len; j++) {                                   /* MHA.h:615-669, padding trimmed :671-682 */
            const int8_t* kj = k_cache + ((size_t)j * kv_heads + kh) * hd;
            int32_t acc = 0;
            for (int d = 0; d < hd; d++) acc += (int32_t)qi[d] * (int32_t)kj[d];
            row[j] = (float)acc * sc->q_s[h] * sc->k_s[kh];               /* quant.h:793-795 */
        }
        softmax_row(row, len, prob);                                      /* Softmax.h:456-635 */
        for (int j = 0; j < len; j++) {                                   /* MHA_i8xi8.h:809 */
            float t = prob[j] / (1.0f * sc->a_s[h]);
            int rt = (int)roundf(t);
            p8[j] = (uint8_t)(rt > 255 ? 255 : rt);
        }
        if (p8_out) memcpy(p8_out + (size_t)h * len, p8, (size_t)len);
        if (o)
            for (int d = 0; d < hd; d++) {
                int32_t acc = 0;                                          /* MHA.h:854-907 */
                for (int j = 0; j < len; j++)
                    acc += (int32_t)p8[j] * (int32_t)v_cache[((size_t)j * kv_heads + kh) * hd + d];
                o[(size_t)h * hd + d] = (float)acc * sc->a_s[h] * sc->v_s[kh]; /* MHA_i8xi8.h:987 */
            }
    }
    free(row); free(prob); free(p8);
    }
}

/* ------------------------------------- attention with dynamic per-(token, head) scales */

/* One row: scores a[0..n) (masked entries -1e32) -> softmax -> fold V's per-token scale -> symmetric dynamic quant
 * (quant.h:578-615 on the row: absmax / 127, 0 -> 1) -> P.V -> dequant.  v8/v_s are indexed [j][kvh]. */
static void dyn_row_tail(const float* row, int n, int n_alloc, const int8_t* v8, const float* v_s, const float* v_ch_s,
                         int kv_heads, int kh, int hd, float* prob, int8_t* p8, float* p_s_out, float* o) {
    (void)n_alloc;
    softmax_row(row, n, prob);
    float vmax = (float)-1e32, vmin = (float)1e32;
    for (int j = 0; j < n; j++) {
        prob[j] = prob[j] * v_s[(size_t)j * kv_heads + kh];
        if (prob[j] > vmax) vmax = prob[j];                               /* quant.h:548-553 */
        if (prob[j] < vmin) vmin = prob[j];
    }
    float amax = fabsf(vmax), amin = fabsf(vmin);
    float sp = (amax > amin ? amax : amin) / 127.0f;                      /* quant.h:600-603 */
    if (sp == 0) sp = 1;
    for (int j = 0; j < n; j++) p8[j] = (int8_t)(int)roundf(prob[j] / sp); /* quant.h:611-612 */
    if (p_s_out) *p_s_out = sp;
    if (o)
        for (int d = 0; d < hd; d++) {
            int32_t acc = 0;
            for (int j = 0; j < n; j++) acc += (int32_t)p8[j] * (int32_t)v8[((size_t)j * kv_heads + kh) * hd + d];
            float t = (float)acc * sp;                                    /* quant.h:646-647 */
            o[d] = v_ch_s ? t * v_ch_s[kh * hd + d] : t;
        }
}

void fxo_mha_prefill_dyn(const float* q, const float* k, const float* v, int s, int q_heads, int kv_heads, int hd,
                         const float* v_ch_s, int8_t* q8_out, float* q_s_out, int8_t* k8_out, float* k_s_out,
                         int8_t* v8_out, float* v_s_out, int8_t* p8_out, float* p_s_out, float* o) {
    const int group = q_heads / kv_heads;
    int8_t* q8 = (int8_t*)malloc((size_t)s * q_heads * hd);
    int8_t* k8 = (int8_t*)malloc((size_t)s * kv_heads * hd);
    int8_t* v8 = (int8_t*)malloc((size_t)s * kv_heads * hd);
    float* qs = (float*)malloc(sizeof(float) * (size_t)s * q_heads);
    float* ks = (float*)malloc(sizeof(float) * (size_t)s * kv_heads);
    float* vs = (float*)malloc(sizeof(float) * (size_t)s * kv_heads);
    fxo_head_quant_sym(q, s, q_heads, hd, 8, q8, qs);
    fxo_head_quant_sym(k, s, kv_heads, hd, 8, k8, ks);
    fxo_head_quant_sym(v, s, kv_heads, hd, 8, v8, vs);
    const float root = sqrtf((float)hd);
    for (int i = 0; i < s * q_heads; i++) qs[i] = qs[i] / root;
#pragma omp parallel
    {
    float* row = (float*)malloc(sizeof(float) * s);
    float* prob = (float*)malloc(sizeof(float) * s);
    int8_t* p8 = (int8_t*)malloc((size_t)s);
#pragma omp for collapse(2) schedule(dynamic, 8)
    for (int h = 0; h < q_heads; h++)
        for (int i = 0; i < s; i++) {
            const int kh = h / group;
            const int8_t* qi = q8 + ((size_t)i * q_heads + h) * hd;
            for (int j = 0; j < s; j++) {
                const int8_t* kj = k8 + ((size_t)j * kv_heads + kh) * hd;
                int32_t acc = 0;
                for (int d = 0; d < hd; d++) acc += (int32_t)qi[d] * (int32_t)kj[d];
                float a = (float)acc * qs[(size_t)i * q_heads + h] * ks[(size_t)j * kv_heads + kh];   /* quant.h:240 */
                row[j] = (j <= i) ? a : (float)-1e32;
            }
            dyn_row_tail(row, s, s, v8, vs, v_ch_s, kv_heads, kh, hd, prob, p8,
                         p_s_out ? p_s_out + (size_t)i * q_heads + h : NULL,
                         o ? o + ((size_t)i * q_heads + h) * hd : NULL);
            if (p8_out) memcpy(p8_out + ((size_t)h * s + i) * s, p8, (size_t)s);
        }
    free(row); free(prob); free(p8);
    }
    if (q8_out) memcpy(q8_out, q8, (size_t)s * q_heads * hd);
    if (k8_out) memcpy(k8_out, k8, (size_t)s * kv_heads * hd);
    if (v8_out) memcpy(v8_out, v8, (size_t)s * kv_heads * hd);
    if (q_s_out) memcpy(q_s_out, qs, sizeof(float) * (size_t)s * q_heads);
    if (k_s_out) memcpy(k_s_out, ks, sizeof(float) * (size_t)s * kv_heads);
    if (v_s_out) memcpy(v_s_out, vs, sizeof(float) * (size_t)s * kv_heads);
    free(q8); free(k8); free(v8); free(qs); free(ks); free(vs);
}

void fxo_mha_decode_dyn(const int8_t* q8, const float* q_s, const int8_t* k_cache, const float* k_s,
                        const int8_t* v_cache, const float* v_s, const float* v_ch_s, int len, int q_heads,
                        int kv_heads, int hd, int8_t* p8_out, float* p_s_out, float* o) {
    const int group = q_heads / kv_heads;
#pragma omp parallel
    {
    float* row = (float*)malloc(sizeof(float) * len);
    float* prob = (float*)malloc(sizeof(float) * len);
    int8_t* p8 = (int8_t*)malloc((size_t)len);
#pragma omp for schedule(static)
    for (int h = 0; h < q_heads; h++) {
        const int kh = h / group;
        const int8_t* qi = q8 + (size_t)h * hd;
        for (int j = 0; j < len; j++) {
            const int8_t* kj = k_cache + ((size_t)j * kv_heads + kh) * hd;
            int32_t acc = 0;
            for (int d = 0; d < hd; d++) acc += (int32_t)qi[d] * (int32_t)kj[d];
            row[j] = (float)acc * q_s[h] * k_s[(size_t)j * kv_heads + kh];
        }
        dyn_row_tail(row, len, len, v_cache, v_s, v_ch_s, kv_heads, kh, hd, prob, p8, p_s_out ? p_s_out + h : NULL,
                     o ? o + (size_t)h * hd : NULL);
        if (p8_out) memcpy(p8_out + (size_t)h * len, p8, (size_t)len);
    }
    free(row); free(prob); free(p8);
    }
}

/* --------------------------------------------------------- fp16 / lm_head */

float fxo_half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else {
            int e = -1;
            do { e++; man <<= 1; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
    else bits = sign | ((exp + 112) << 23) | (man << 13);
    float f; memcpy(&f, &bits, 4); return f;
}

void fxo_embed(const uint16_t* table, int hidden, int token, float* y) {
    for (int k = 0; k < hidden; k++) y[k] = fxo_half_to_float(table[(size_t)token * hidden + k]);
}

void fxo_lm_head(const uint16_t* table, int vocab, int hidden, const float* n, float* logits) {
#pragma omp parallel for schedule(static)
    for (int v = 0; v < vocab; v++) {
        float acc = 0;
        for (int k = 0; k < hidden; k++) acc += fxo_half_to_float(table[(size_t)v * hidden + k]) * n[k];
        logits[v] = acc;
    }
}

int fxo_argmax(const float* x, int n) {
    int best = 0;
    for (int i = 1; i < n; i++) if (x[i] > x[best]) best = i;
    return best;
}

/* Top-k sampling of the next token, Modules/Logits.h:145-279 (dec_Sampling_Embedding_Layer), with the insertion
 * routine of Modules/Logits.h:5-31 (sort_top_k: strict '>', so of two equal logits the one inserted first keeps
 * the higher rank).  `lanes` = block_parallel_samp: lane i scans the contiguous index range
 * [i*n/lanes, (i+1)*n/lanes) in order (Logits.h:216, inner_block_parallel = 1), the per-lane lists are merged
 * rank-major (Logits.h:224-232); softmax over the k candidates with two partial sums (Logits.h:239-254); CDF
 * and "first k with rand < cdf[k]" (Logits.h:258-275).  n % lanes == 0, top_k <= 16.
 * Outputs (each optional): the k candidates, their probabilities; returns the sampled token id. */
static void fxo_sort_top_k(int* idx, float* val, int top_k, int v_idx, float v) {
    int insert_pos = top_k;
    for (int k = 0; k < top_k; k++)
        if (v > val[k] && insert_pos == top_k) insert_pos = k;
    for (int k = top_k - 1; k >= 0; k--) {
        if (k > insert_pos) { idx[k] = idx[k - 1]; val[k] = val[k - 1]; }
        else if (k == insert_pos) { idx[k] = v_idx; val[k] = v; }
    }
}

int fxo_sample_topk(const float* logits, int n, int top_k, int lanes, float rand_seed, int enable_sub_max,
                    int* top_idx, float* top_val, float* top_prob) {
    int* lidx = (int*)malloc(sizeof(int) * (size_t)lanes * top_k);
    float* lval = (float*)malloc(sizeof(float) * (size_t)lanes * top_k);
    int fidx[16]; float fval[16], prob[16], cdf[16];
    for (int i = 0; i < lanes * top_k; i++) { lidx[i] = -1; lval[i] = -1e32f; }
    for (int k = 0; k < top_k; k++) { fidx[k] = -1; fval[k] = -1e32f; }
    const int per = n / lanes;
    for (int m = 0; m < per; m++)
        for (int i = 0; i < lanes; i++)
            fxo_sort_top_k(lidx + (size_t)i * top_k, lval + (size_t)i * top_k, top_k, i * per + m, logits[i * per + m]);
    for (int K = 0; K < top_k; K++)
        for (int i = 0; i < lanes; i++)
            fxo_sort_top_k(fidx, fval, top_k, lidx[(size_t)i * top_k + K], lval[(size_t)i * top_k + K]);
    float sum_partial[2] = {0.0f, 0.0f};
    for (int k = 0; k < top_k; k++) {
        const float t = enable_sub_max ? expf(fval[k] - fval[0]) : expf(fval[k]);
        prob[k] = t;
        sum_partial[k % 2] += t;
    }
    const float sum = sum_partial[0] + sum_partial[1];
    for (int k = 0; k < top_k; k++) prob[k] /= sum;
    cdf[0] = prob[0];
    for (int k = 1; k < top_k; k++) cdf[k] = prob[k] + cdf[k - 1];
    int selected_k = top_k - 1;
    for (int k = 0; k < top_k; k++)
        if (rand_seed < cdf[k] && selected_k == top_k - 1) selected_k = k;
    for (int k = 0; k < top_k; k++) {
        if (top_idx) top_idx[k] = fidx[k];
        if (top_val) top_val[k] = fval[k];
        if (top_prob) top_prob[k] = prob[k];
    }
    free(lidx); free(lval);
    return fidx[selected_k];
}

/* ------------------------------------------------------ layer / model graphs */

static void linear_w8a8(const float* x, int rows, int k, int n, const int8_t* w, const float* ws, float* y) {
    /* quant.h:6 -> Linear_Layer.h:293/862 -> quant.h:115/470, symmetric int8 instantiation */
    int8_t* q = (int8_t*)malloc((size_t)rows * k);
    float* s = (float*)malloc(sizeof(float) * rows);
    int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)rows * n);
    fxo_quant_sym(x, rows, k, 8, q, s);
    fxo_linear_i8(q, w, rows, k, n, acc);
    fxo_dequant(acc, rows, n, s, NULL, ws, NULL, y);
    free(q); free(s); free(acc);
}

static void ffn_block(const fxo_model* m, int l, const float* res0, int rows, int decode, float* res1) {
    const int H = m->hidden, I = m->inter;
    float* n1 = (float*)malloc(sizeof(float) * (size_t)rows * H);
    float* g = (float*)malloc(sizeof(float) * (size_t)rows * I);
    float* u = (float*)malloc(sizeof(float) * (size_t)rows * I);
    float* d = (float*)malloc(sizeof(float) * (size_t)rows * H);
    const float* gamma = m->gamma + (size_t)(2 * l + 1) * H;
    if (decode) fxo_rmsnorm_dec(res0, gamma, H, 8, m->eps, n1);          /* T_BLOCK_PARALLEL=8 */
    else fxo_rmsnorm_pref(res0, gamma, rows, H, m->eps, n1);
    linear_w8a8(n1, rows, H, I, m->wg[l], m->sg[l], g);
    linear_w8a8(n1, rows, H, I, m->wu[l], m->su[l], u);
    fxo_swish(g, rows * I, g);                                           /* SpinQuant_Prefilling.h:1017 */
    fxo_gate(u, g, rows * I, g);                                         /* :1029 up * silu(gate) */
    fxo_fht(g, rows, I, m->fht_scale, u);                                /* :673-684 R4 */
    linear_w8a8(u, rows, I, H, m->wd[l], m->sd[l], d);
    fxo_residual(d, res0, rows * H, res1);
    free(n1); free(g); free(u); free(d);
}

void fxo_llama_decode_token(const fxo_model* m, const float* x_in, int pos, int8_t* k_cache,
                            int8_t* v_cache, float* hidden_out, float* logits) {
    const int H = m->hidden, KV = m->kv_hidden, hd = m->head_dim;
    float* x = (float*)malloc(sizeof(float) * H);
    float* n0 = (float*)malloc(sizeof(float) * H);
    float* q = (float*)malloc(sizeof(float) * H);
    float* k = (float*)malloc(sizeof(float) * KV);
    float* v = (float*)malloc(sizeof(float) * KV);
    float* att = (float*)malloc(sizeof(float) * H);
    float* ao = (float*)malloc(sizeof(float) * H);
    float* res0 = (float*)malloc(sizeof(float) * H);
    int8_t* q8 = (int8_t*)malloc(H);
    memcpy(x, x_in, sizeof(float) * H);
    for (int l = 0; l < m->layers; l++) {
        fxo_mha_scales sc = { m->q_s + (size_t)l * m->q_heads, m->k_s + (size_t)l * m->kv_heads,
                              m->v_s + (size_t)l * m->kv_heads, m->a_s + (size_t)l * m->q_heads };
        int8_t* kc = k_cache + (size_t)l * m->max_pos * KV;
        int8_t* vc = v_cache + (size_t)l * m->max_pos * KV;
        fxo_rmsnorm_dec(x, m->gamma + (size_t)(2 * l) * H, H, 8, m->eps, n0);
        linear_w8a8(n0, 1, H, KV, m->wk[l], m->sk[l], k);
        linear_w8a8(n0, 1, H, KV, m->wv[l], m->sv[l], v);
        linear_w8a8(n0, 1, H, H, m->wq[l], m->sq[l], q);
        fxo_rope(k, 1, m->kv_heads, hd, m->rope_sin, m->rope_cos, pos, k);   /* Decoding_mem_opt.h:698 */
        fxo_rope(q, 1, m->q_heads, hd, m->rope_sin, m->rope_cos, pos, q);    /* :707 */
        fxo_static_quant(k, 1, m->kv_heads, hd, sc.k_s, 1.0f, 1, 8, kc + (size_t)pos * KV); /* :738 */
        fxo_static_quant(v, 1, m->kv_heads, hd, sc.v_s, 1.0f, 1, 8, vc + (size_t)pos * KV); /* :742 */
        fxo_static_quant(q, 1, m->q_heads, hd, sc.q_s, sqrtf((float)hd), 1, 8, q8);         /* :746 */
        fxo_mha_decode(q8, kc, vc, pos + 1, m->q_heads, m->kv_heads, hd, &sc, NULL, att);
        linear_w8a8(att, 1, H, H, m->wo[l], m->so[l], ao);
        fxo_residual(ao, x, H, res0);
        ffn_block(m, l, res0, 1, 1, x);
    }
    if (hidden_out) memcpy(hidden_out, x, sizeof(float) * H);
    if (logits) {
        fxo_rmsnorm_dec(x, m->gamma + (size_t)(2 * m->layers) * H, H, 8, m->eps, n0);
        fxo_lm_head(m->embed, m->vocab, H, n0, logits);
    }
    free(x); free(n0); free(q); free(k); free(v); free(att); free(ao); free(res0); free(q8);
}

void fxo_llama_prefill(const fxo_model* m, const float* x_in, int s, int8_t* k_cache, int8_t* v_cache,
                       float* hidden_out) {
    const int H = m->hidden, KV = m->kv_hidden, hd = m->head_dim;
    float* x = (float*)malloc(sizeof(float) * (size_t)s * H);
    float* n0 = (float*)malloc(sizeof(float) * (size_t)s * H);
    float* q = (float*)malloc(sizeof(float) * (size_t)s * H);
    float* k = (float*)malloc(sizeof(float) * (size_t)s * KV);
    float* v = (float*)malloc(sizeof(float) * (size_t)s * KV);
    float* att = (float*)malloc(sizeof(float) * (size_t)s * H);
    float* ao = (float*)malloc(sizeof(float) * (size_t)s * H);
    float* res0 = (float*)malloc(sizeof(float) * (size_t)s * H);
    memcpy(x, x_in, sizeof(float) * (size_t)s * H);
    for (int l = 0; l < m->layers; l++) {
        fxo_mha_scales sc = { m->q_s + (size_t)l * m->q_heads, m->k_s + (size_t)l * m->kv_heads,
                              m->v_s + (size_t)l * m->kv_heads, m->a_s + (size_t)l * m->q_heads };
        int8_t* kc = k_cache + (size_t)l * m->max_pos * KV;
        int8_t* vc = v_cache + (size_t)l * m->max_pos * KV;
        fxo_rmsnorm_pref(x, m->gamma + (size_t)(2 * l) * H, s, H, m->eps, n0);
        linear_w8a8(n0, s, H, KV, m->wk[l], m->sk[l], k);
        linear_w8a8(n0, s, H, H, m->wq[l], m->sq[l], q);
        linear_w8a8(n0, s, H, KV, m->wv[l], m->sv[l], v);
        fxo_rope(k, s, m->kv_heads, hd, m->rope_sin, m->rope_cos, 0, k);
        fxo_rope(q, s, m->q_heads, hd, m->rope_sin, m->rope_cos, 0, q);
        fxo_mha_prefill(q, k, v, s, m->q_heads, m->kv_heads, hd, &sc, NULL, kc, vc, NULL, att);
        linear_w8a8(att, s, H, H, m->wo[l], m->so[l], ao);
        fxo_residual(ao, x, s * H, res0);
        ffn_block(m, l, res0, s, 0, x);
    }
    if (hidden_out) memcpy(hidden_out, x, sizeof(float) * (size_t)s * H);
    free(x); free(n0); free(q); free(k); free(v); free(att); free(ao); free(res0);
}

/* ---------------------------------------------------------- data_io.h layouts */

void fxo_pack_pref(const float* x, int tokens, int dim, int tp, float* packed) {
    for (int t = 0; t < tokens; t++)                                      /* data_io.h:15-19 */
        for (int k = 0; k < dim; k++) packed[((size_t)(t / tp) * dim + k) * tp + t % tp] = x[(size_t)t * dim + k];
}
void fxo_unpack_pref(const float* packed, int tokens, int dim, int tp, float* x) {
    for (int t = 0; t < tokens; t++)
        for (int k = 0; k < dim; k++) x[(size_t)t * dim + k] = packed[((size_t)(t / tp) * dim + k) * tp + t % tp];
}
void fxo_pack_dec(const float* x, int dim, int bp, float* packed) {
    const int per = dim / bp;                                             /* Linear_Layer_Decoding_tb.cpp:148 */
    for (int f = 0; f < dim; f++) packed[(size_t)(f % per) * bp + f / per] = x[f];
}
void fxo_unpack_dec(const float* packed, int dim, int bp, float* x) {
    const int per = dim / bp;
    for (int f = 0; f < dim; f++) x[f] = packed[(size_t)(f % per) * bp + f / per];
}

// Shared device helpers and host-side error plumbing for libflexllm_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/flexllm_hip.h"

namespace fx {

constexpr int kWave = 64;

using i32x4 = int __attribute__((ext_vector_type(4)));
using i32x16 = int __attribute__((ext_vector_type(16)));
using f32x4 = float __attribute__((ext_vector_type(4)));

void set_error(const char* fmt, ...);

#define FX_REQUIRE(cond, ...)                                   \
    do {                                                        \
        if (!(cond)) {                                          \
            fx::set_error(__VA_ARGS__);                         \
            return FLEXLLM_EINVAL;                              \
        }                                                       \
    } while (0)

#define FX_HIP(call)                                                                   \
    do {                                                                               \
        hipError_t e_ = (call);                                                        \
        if (e_ != hipSuccess) {                                                        \
            fx::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
            return FLEXLLM_EHIP;                                                       \
        }                                                                              \
    } while (0)

#define FX_LAUNCH_CHECK()                                                              \
    do {                                                                               \
        hipError_t e_ = hipGetLastError();                                             \
        if (e_ != hipSuccess) {                                                        \
            fx::set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(e_), __FILE__, __LINE__); \
            return FLEXLLM_EHIP;                                                       \
        }                                                                              \
    } while (0)

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Scratch of the stand-alone entry points that need device memory beyond their arguments (arg-max and top-k
// candidates, decode attention's scores / statistics / accumulators).  One buffer per (device, stream, kind), at least
// `bytes` long and 256-byte aligned, allocated on first use and grown on demand: work of one stream runs in order and
// may share a buffer, calls on different streams get different buffers and may run at the same time (also from
// several host threads).  Growing waits for the stream's earlier work before the old buffer is freed.  A buffer is
// released when its stream is destroyed through flexllm_rt_stream_destroy, otherwise it lives until the process ends.
enum ScratchKind { kScratchArgmax = 0, kScratchTopK = 1, kScratchMhaDecode = 2, kScratchMhaDecodeDyn = 3 };
int stream_scratch(ScratchKind kind, hipStream_t st, size_t bytes, void** out);
void stream_scratch_release(hipStream_t st);

// ---------------------------------------------------------------- cross-lane exchange
// Value held by lane (lane ^ MASK).  1,2: DPP quad_perm; 8: DPP row rotate by 8; 4: two DPP row shifts, each
// writing the banks (groups of four lanes) it is right for; 16: ds_swizzle bit mode (no LDS traffic, crossbar
// only); 32: bpermute.  The DPP forms are plain VALU moves which the compiler folds into the consuming add.
template <int MASK>
__device__ __forceinline__ int lane_xor_i(int v) {
    if constexpr (MASK == 1) {
        return __builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
    } else if constexpr (MASK == 2) {
        return __builtin_amdgcn_mov_dpp(v, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    } else if constexpr (MASK == 4) {
        const int lo = __builtin_amdgcn_update_dpp(v, v, 0x104, 0xF, 0x5, false);   // row_shl:4 into banks 0,2: lane i <- i+4
        return __builtin_amdgcn_update_dpp(lo, v, 0x114, 0xF, 0xA, false);          // row_shr:4 into banks 1,3: lane i <- i-4
    } else if constexpr (MASK == 8) {
        return __builtin_amdgcn_mov_dpp(v, 0x128, 0xF, 0xF, true);  // row_ror:8
    } else if constexpr (MASK == 16) {
        return __builtin_amdgcn_ds_swizzle(v, (MASK << 10) | 0x1F); // and=0x1f or=0 xor=MASK
    } else {
        static_assert(MASK == 32, "lane_xor mask");
        return __builtin_amdgcn_ds_bpermute(((int)(threadIdx.x & 63) ^ 32) << 2, v);
    }
}
template <int MASK>
__device__ __forceinline__ float lane_xor_f(float v) {
    return __int_as_float(lane_xor_i<MASK>(__float_as_int(v)));
}
// Butterfly across lanes: the lane whose MASK bit is clear gets a + p, the other p - a, with p the partner's value.
// `sign` is 0 or 0x80000000 by that bit: p + (+-a) is the same IEEE sum or difference, in one add.
template <int MASK>
__device__ __forceinline__ unsigned lane_sign(int lane) { return (lane & MASK) ? 0x80000000u : 0u; }
template <int MASK>
__device__ __forceinline__ float lane_butterfly_s(float a, unsigned sign) {
    return lane_xor_f<MASK>(a) + __int_as_float(__float_as_int(a) ^ (int)sign);
}

// x / d for a divisor used many times, r = 1.0f / d: the product x*r is within an ulp of the quotient, its exact
// residual (one fma) corrects it, and the corrected value is the correctly rounded quotient whenever r is the
// correctly rounded reciprocal and nothing under- or overflows (Markstein).  Callers keep |x| within
// [2^-60, 2^100] or fall back to the division (`div_fast_ok` on the largest magnitude they divide).
__device__ __forceinline__ float div_fast(float x, float d, float r) {
    const float q = x * r;
    return __builtin_fmaf(__builtin_fmaf(-q, d, x), r, q);
}
__device__ __forceinline__ bool div_fast_ok(float amax, float d) {
    return amax >= 0x1p-60f && amax <= 0x1p100f && d >= 0x1p-20f && d <= 0x1p20f;
}

// e^x on the hardware's 2^x unit (1 ulp).  The exponent x*log2(e) is formed in two parts: t is the rounded
// product, lo its rounding error plus the low part of log2(e), folded back as e*(1 + lo*ln2).  Result within about
// 2 ulp of the correctly rounded value for any x whose result is a normal number; t is capped so that 2^t stays
// finite (callers pass x <= 0 or take 1/(1+e^x), where a cap at 2^126 changes nothing representable).
template <bool CLAMP = true>                     // CLAMP = false for callers that guarantee x <= 0
__device__ __forceinline__ float exp_f(float x) {
    const float t = x * 1.44269502162933349609375f;
    const float lo = __builtin_fmaf(x, 1.92596299e-8f, __builtin_fmaf(x, 1.44269502162933349609375f, -t));
    const float e = __builtin_amdgcn_exp2f(CLAMP ? fminf(t, 126.0f) : t);
    return __builtin_fmaf(e, lo * 0.693147182464599609375f, e);
}
// SiLU x / (1 + exp(-x)) with the hardware reciprocal (1 ulp) in place of the division: within 4 ulp of the
// reference's value.  Every kernel that applies SiLU calls this one function, so they agree bit for bit.
__device__ __forceinline__ float silu_f(float v) { return v * __builtin_amdgcn_rcpf(1.0f + exp_f(-v)); }

// Wave-wide reductions; every lane gets the result.  Inside a row of 16 lanes: the xor butterfly on DPP moves.  Across
// the four rows: two DPP row broadcasts (lane 15 of rows 0 and 2 into rows 1 and 3, then lane 31 into rows 2 and 3)
// leave the total in lane 63, which a readlane hands to all lanes as a scalar.  The operands of each addition are the
// ones the full butterfly (xor 16, xor 32) pairs in lane 63, so sums keep their bits; the row broadcasts are ordinary
// VALU moves, where the swizzle and the bpermute of the butterfly each take a trip through the LDS pipe.
__device__ __forceinline__ int row_bcast15_i(int v, int keep) { return __builtin_amdgcn_update_dpp(keep, v, 0x142, 0xA, 0xF, false); }
__device__ __forceinline__ int row_bcast31_i(int v, int keep) { return __builtin_amdgcn_update_dpp(keep, v, 0x143, 0xC, 0xF, false); }
__device__ __forceinline__ float row_bcast15_f(float v, float keep) { return __int_as_float(row_bcast15_i(__float_as_int(v), __float_as_int(keep))); }
__device__ __forceinline__ float row_bcast31_f(float v, float keep) { return __int_as_float(row_bcast31_i(__float_as_int(v), __float_as_int(keep))); }
__device__ __forceinline__ float lane63_f(float v) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63)); }

__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, lane_xor_f<1>(v));
    v = fmaxf(v, lane_xor_f<2>(v));
    v = fmaxf(v, lane_xor_f<4>(v));
    v = fmaxf(v, lane_xor_f<8>(v));
    v = fmaxf(v, row_bcast15_f(v, v));               // rows the broadcast does not write keep their own value
    v = fmaxf(v, row_bcast31_f(v, v));
    return lane63_f(v);
}
__device__ __forceinline__ float wave_min(float v) {
    v = fminf(v, lane_xor_f<1>(v));
    v = fminf(v, lane_xor_f<2>(v));
    v = fminf(v, lane_xor_f<4>(v));
    v = fminf(v, lane_xor_f<8>(v));
    v = fminf(v, row_bcast15_f(v, v));
    v = fminf(v, row_bcast31_f(v, v));
    return lane63_f(v);
}
__device__ __forceinline__ float wave_sum(float v) {
    v += lane_xor_f<1>(v);
    v += lane_xor_f<2>(v);
    v += lane_xor_f<4>(v);
    v += lane_xor_f<8>(v);
    v += row_bcast15_f(v, 0.0f);                     // lane 63's row is written by both broadcasts: it never adds the 0
    v += row_bcast31_f(v, 0.0f);
    return lane63_f(v);
}
__device__ __forceinline__ int wave_sum_i(int v) {
    v += lane_xor_i<1>(v);
    v += lane_xor_i<2>(v);
    v += lane_xor_i<4>(v);
    v += lane_xor_i<8>(v);
    v += row_bcast15_i(v, 0);
    v += row_bcast31_i(v, 0);
    return __builtin_amdgcn_readlane(v, 63);
}

// Block-wide reductions for blocks of NW waves; `red` is NW floats of LDS.  Every thread gets the result.
template <int NW>
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    if constexpr (NW == 1) return v;
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r = fmaxf(r, red[i]);
    return r;
}
template <int NW>
__device__ __forceinline__ float block_min(float v, float* red) {
    v = wave_min(v);
    if constexpr (NW == 1) return v;
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r = fminf(r, red[i]);
    return r;
}
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    if constexpr (NW == 1) return v;
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r += red[i];
    return r;
}

// ---------------------------------------------------------------- quantisation arithmetic
// round half away from zero of x/s with IEEE division, wrapped to 8 bits like (ap_int<8>)round(x/s).
__device__ __forceinline__ int quant_round(float x, float s) { return (int)roundf(x / s); }

// round(x / s) for a whole vector that shares s, without a division per element.  q~ = x * rcp(s) is within
// 4 * 2^-24 * |q| <= 3.1e-5 of the correctly rounded quotient for |q| <= 127.5 (symmetric int8), <= 6.1e-5 for
// |q| <= 255 (the asymmetric uint8 use: still inside the window, with a margin of 1.6), so both round to the same integer
// unless q~ lies within 1e-4 of a tie (k + 0.5); `near_tie` collects those cases and the caller redoes them
// with the exact expression.  Valid while 1/s is a normal number (`quant_fast_ok`).
__device__ __forceinline__ bool quant_fast_ok(float s) { return s >= 0x1p-100f && s <= 0x1p100f; }
__device__ __forceinline__ int quant_round_fast(float x, float rs, bool& near_tie) {
    const float q = x * rs;
    const float r = __builtin_rintf(q);              // nearest integer (ties to even: a tie is redone by the caller anyway)
    near_tie |= fabsf(q - r) > 0.4999f;              // within 1e-4 of k + 0.5
    return (int)r;
}
template <int N>
__device__ __forceinline__ void quant_vector(const float (&v)[N], float s, int (&n)[N]) {
    if (!quant_fast_ok(s)) {
#pragma unroll
        for (int i = 0; i < N; i++) n[i] = quant_round(v[i], s);
        return;
    }
    const float rs = __builtin_amdgcn_rcpf(s);       // 1 ulp: the product below is then within 4 * 2^-24 * |q| of the quotient
    constexpr int G = N % 4 == 0 ? 4 : N;            // the exact path is taken per group: rare (about 2e-4 per element)
#pragma unroll
    for (int g = 0; g < N / G; g++) {
        bool redo = false;
#pragma unroll
        for (int i = 0; i < G; i++) n[g * G + i] = quant_round_fast(v[g * G + i], rs, redo);
        if (redo) {
#pragma unroll
            for (int i = 0; i < G; i++) n[g * G + i] = quant_round(v[g * G + i], s);
        }
    }
}

__device__ __forceinline__ uint32_t pack4_i8(int a, int b, int c, int d) {
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) | ((uint32_t)(d & 0xff) << 24);
}

// symmetric scale from a row's absmax: absmax/127, 0 -> 1
__device__ __forceinline__ float sym_scale(float absmax, float scale_base) {
    float s = absmax / scale_base;
    return s == 0.0f ? 1.0f : s;
}
// The same for a maximum that every lane of the wave holds (the result of a block-wide reduction), int8 range: the
// division by 127 goes through the correctly rounded reciprocal and one exact residual step (`div_fast`), which gives
// the IEEE quotient for every float32 in the guarded range (all 2^23 significands checked against the division on the
// CPU; the sequence does not depend on the exponent while nothing under- or overflows), behind a scalar branch so that
// the long division sequence is not issued as well.
__device__ __forceinline__ float sym_scale_127_uniform(float absmax) {
    constexpr float r127 = 1.0f / 127.0f;            // correctly rounded at compile time
    float s;
    if (__builtin_amdgcn_readfirstlane((int)(absmax >= 0x1p-60f && absmax <= 0x1p100f))) s = div_fast(absmax, 127.0f, r127);
    else s = absmax / 127.0f;
    return s == 0.0f ? 1.0f : s;
}

}  // namespace fx

// Fast Walsh-Hadamard transform of fp32 rows (SpinQuant online rotation), optionally fused with the
// per-token int8 quantisation that follows it.
//
// The reference runs an omega network: log2(n) x (perfect shuffle, butterfly on adjacent pairs).  That is
// the in-place butterfly network whose stage s pairs the elements whose indices differ in bit
// (s+1) mod log2(n), the bit-clear element receiving u+v and the bit-set element u-v.  Running the
// stages in that order (bits 1,2,...,log2(n)-1, then 0) reproduces the reference's fp32 result bit for
// bit, so the int8 tensor quantised from it is exact as well.
//
// One workgroup of 256 threads transforms one row of n = 256 * NR elements, NR = 2^P values per thread:
//   layout A: element i = j*1024 + t*4 + e   (float4 loads; e = bits 0-1, t = bits 2-9, j = bits 10+)
//             -> stage bit 1 in registers, bits 2..7-P as cross-lane butterflies on lane bits 0..5-P (DPP only:
//             one stage at n = 8192, four at n = 1024)
//   through LDS to layout M: i = hi*256 + r*2^(8-P) + lo, thread = (hi, lo), r = bits 8-P..7
//             -> stages bits 8-P..7 in registers
//   through LDS to layout B: i = r*256 + t   (r = bits 8+, t = bits 0-7)
//             -> stages bits 8.. in registers, then bit 0 as a DPP butterfly.
// A butterfly between registers is one add or subtract; across lanes it costs a data movement as well, so all but a
// few stages run between registers, at the price of a second pass through LDS.  Each 256-element block of the LDS row
// is followed by 2^(8-P) floats of padding, which spreads layout M's reads over all banks.
#pragma once
#include "common.h"

namespace fx {

constexpr int kFhtBlock = 256;

// QUANT: 0 = fp32 output y; 1 = per-row symmetric int8 (q, s); 2 = per-row asymmetric quantisation to scale_base steps
// (uint4: 15), one value per byte, with the scale in s and the row minimum in zp - what quant_asym_kernel computes from
// the fp32 output, to the bit.
template <int LOG2N, int QUANT, bool SWIGLU = false>
__global__ __launch_bounds__(kFhtBlock) void fht_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                        int8_t* __restrict__ q, float* __restrict__ s, float scale,
                                                        float* __restrict__ zp = nullptr, float scale_base = 15.0f,
                                                        unsigned mask = 15u) {
    constexpr int N = 1 << LOG2N;
    constexpr int NJ = N / 1024;   // float4 vectors per thread in layout A
    constexpr int NR = N / 256;    // floats per thread in layouts M and B
    constexpr int P = LOG2N - 8;   // log2(NR)
    constexpr int PAD = 1 << (8 - P);
    static_assert(P >= 2 && P <= 5, "1024 <= n <= 8192");
    __shared__ float lds[N + PAD * NR];
    __shared__ float red[kFhtBlock / kWave];
    const int t = threadIdx.x;
    const int lane = t & 63;
    const size_t row = blockIdx.x;
    float4 a[NJ];
    if constexpr (SWIGLU) {
        // input row is [2N] interleaved (gate_i, up_i); element i = up_i * silu(gate_i)
        const float4* xr = reinterpret_cast<const float4*>(x + row * (2 * N));
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const float4 p0 = xr[(j * 256 + t) * 2], p1 = xr[(j * 256 + t) * 2 + 1];
            a[j].x = p0.y * silu_f(p0.x);
            a[j].y = p0.w * silu_f(p0.z);
            a[j].z = p1.y * silu_f(p1.x);
            a[j].w = p1.w * silu_f(p1.z);
        }
    } else {
        const float4* xr = reinterpret_cast<const float4*>(x + row * N);
#pragma unroll
        for (int j = 0; j < NJ; j++) a[j] = xr[j * 256 + t];
    }

    // stage: bit 1 (elements e and e^2 of each float4)
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const float u0 = a[j].x, v0 = a[j].z, u1 = a[j].y, v1 = a[j].w;
        a[j].x = u0 + v0; a[j].z = u0 - v0;
        a[j].y = u1 + v1; a[j].w = u1 - v1;
    }
    // stages: bits 2..7-P = lane bits 0..5-P
#define FX_LANE_STAGE(MASK)                                             \
    {                                                                   \
        const unsigned sg = lane_sign<MASK>(lane);                      \
        _Pragma("unroll") for (int j = 0; j < NJ; j++) {                \
            a[j].x = lane_butterfly_s<MASK>(a[j].x, sg);                \
            a[j].y = lane_butterfly_s<MASK>(a[j].y, sg);                \
            a[j].z = lane_butterfly_s<MASK>(a[j].z, sg);                \
            a[j].w = lane_butterfly_s<MASK>(a[j].w, sg);                \
        }                                                               \
    }
    FX_LANE_STAGE(1)
    if constexpr (P < 5) FX_LANE_STAGE(2)
    if constexpr (P < 4) FX_LANE_STAGE(4)
    if constexpr (P < 3) FX_LANE_STAGE(8)
#undef FX_LANE_STAGE

    // A -> M through LDS (float4 stores: conflict-free whatever the padding)
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int i = j * 1024 + t * 4;
        *reinterpret_cast<float4*>(&lds[i + PAD * (i >> 8)]) = a[j];
    }
    __syncthreads();
    float b[NR];
    {
        constexpr int LOB = 8 - P;                               // low index bits that stay with the thread
        const int base = (t >> LOB) * (256 + PAD) + (t & ((1 << LOB) - 1));
#pragma unroll
        for (int r = 0; r < NR; r++) b[r] = lds[base + (r << LOB)];
        // stages: bits 8-P..7 = register index bits 0..P-1
#pragma unroll
        for (int bit = 1; bit < NR; bit <<= 1) {
#pragma unroll
            for (int r = 0; r < NR; r++) {
                if ((r & bit) == 0) {
                    const float u = b[r], v = b[r | bit];
                    b[r] = u + v;
                    b[r | bit] = u - v;
                }
            }
        }
        // every thread rewrites exactly the slots it read, so no barrier is needed before these stores
#pragma unroll
        for (int r = 0; r < NR; r++) lds[base + (r << LOB)] = b[r];
    }
    __syncthreads();
    // M -> B
#pragma unroll
    for (int r = 0; r < NR; r++) b[r] = lds[r * (256 + PAD) + t];

    // stages: bits 8..LOG2N-1 = register index bits 0..
#pragma unroll
    for (int bit = 1; bit < NR; bit <<= 1) {
#pragma unroll
        for (int r = 0; r < NR; r++) {
            if ((r & bit) == 0) {
                const float u = b[r], v = b[r | bit];
                b[r] = u + v;
                b[r | bit] = u - v;
            }
        }
    }
    // last stage: bit 0 = lane bit 0
    {
        const unsigned sg = lane_sign<1>(lane);
#pragma unroll
        for (int r = 0; r < NR; r++) b[r] = lane_butterfly_s<1>(b[r], sg);
    }

    float amax = 0.0f;
    if constexpr (QUANT == 0) {
#pragma unroll
        for (int r = 0; r < NR; r++) b[r] = b[r] / scale;
    } else {
        // b / scale through the reciprocal with an exact residual step: the correctly rounded quotient for every
        // magnitude this thread holds, or the plain division when its largest one is outside the safe range
        // (smaller elements of a thread that passes quantise to zero under either form).  Division by a
        // positive constant is monotonic, so the largest quotient is the quotient of the largest magnitude.
#pragma unroll
        for (int r = 0; r < NR; r++) amax = fmaxf(amax, fabsf(b[r]));
        if (div_fast_ok(amax, scale)) {
            const float rs = 1.0f / scale;
#pragma unroll
            for (int r = 0; r < NR; r++) b[r] = div_fast(b[r], scale, rs);
        } else {
#pragma unroll
            for (int r = 0; r < NR; r++) b[r] = b[r] / scale;
        }
        amax = amax / scale;
    }
    if constexpr (QUANT == 0) {
        float* yr = y + row * N;
#pragma unroll
        for (int r = 0; r < NR; r++) yr[r * 256 + t] = b[r];
    } else if constexpr (QUANT == 2) {
        // the quotients above are the fp32 outputs (correctly rounded either way); their extremes, then
        // round((v - min) / s) & mask as quant_asym_kernel forms it
        float vmax = b[0], vmin = b[0];
#pragma unroll
        for (int r = 1; r < NR; r++) { vmax = fmaxf(vmax, b[r]); vmin = fminf(vmin, b[r]); }
        vmax = block_max<kFhtBlock / kWave>(vmax, red);   // its leading barrier also retires the lds reads above
        vmin = block_min<kFhtBlock / kWave>(vmin, red);
        float sc = (vmax - vmin) / scale_base;
        if (sc == 0.0f) sc = 1.0f;
        if (t == 0) { s[row] = sc; zp[row] = vmin; }
        uint8_t* lds_q = reinterpret_cast<uint8_t*>(lds);
        {
            float d[NR];
            int nq[NR];
#pragma unroll
            for (int r = 0; r < NR; r++) d[r] = b[r] - vmin;
            quant_vector(d, sc, nq);
#pragma unroll
            for (int r = 0; r < NR; r++) lds_q[r * 256 + t] = (uint8_t)(nq[r] & mask);
        }
        __syncthreads();
        i32x4* qr = reinterpret_cast<i32x4*>(q + row * N);
        for (int c = t; c < N / 16; c += kFhtBlock) qr[c] = reinterpret_cast<const i32x4*>(lds_q)[c];
    } else {
        amax = block_max<kFhtBlock / kWave>(amax, red);   // its leading barrier also retires the lds reads above
        const float sc = sym_scale_127_uniform(amax);
        if (t == 0) s[row] = sc;
        int8_t* lds_q = reinterpret_cast<int8_t*>(lds);
        {
            int nq[NR];
            quant_vector(b, sc, nq);          // x * (1/s) with the exact x / s near rounding ties: same integers
#pragma unroll
            for (int r = 0; r < NR; r++) lds_q[r * 256 + t] = (int8_t)nq[r];
        }
        __syncthreads();
        i32x4* qr = reinterpret_cast<i32x4*>(q + row * N);
        for (int c = t; c < N / 16; c += kFhtBlock) qr[c] = reinterpret_cast<const i32x4*>(lds_q)[c];
    }
}

template <int QUANT>
static int launch_fht(const float* x, float* y, int8_t* q, float* s, int rows, int n, float scale, hipStream_t st,
                      float* zp = nullptr, float scale_base = 15.0f, unsigned mask = 15u) {
    switch (n) {
        case 1024: fht_kernel<10, QUANT><<<rows, kFhtBlock, 0, st>>>(x, y, q, s, scale, zp, scale_base, mask); break;
        case 2048: fht_kernel<11, QUANT><<<rows, kFhtBlock, 0, st>>>(x, y, q, s, scale, zp, scale_base, mask); break;
        case 4096: fht_kernel<12, QUANT><<<rows, kFhtBlock, 0, st>>>(x, y, q, s, scale, zp, scale_base, mask); break;
        case 8192: fht_kernel<13, QUANT><<<rows, kFhtBlock, 0, st>>>(x, y, q, s, scale, zp, scale_base, mask); break;
        default:
            set_error("fht: n=%d must be a power of two in [1024, 8192]", n);
            return FLEXLLM_EINVAL;
    }
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx

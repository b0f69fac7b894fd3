// int8 x int8 -> int32 GEMM for prefill on gfx950 matrix cores: C[m][n] = sum_k A[m][k]*W[n][k].
//
// Both operands are K-contiguous, which is exactly the per-lane operand shape of
// v_mfma_i32_32x32x32_i8 (lane l supplies 16 consecutive k-bytes of row/column l%32, k-group l/32), so
// tiles go global -> registers -> LDS (16-byte chunks, k-chunk-major planes) -> MFMA operands with plain
// 128-bit reads and no transposition.  Integer accumulation: exact in any order.
//
// Workgroup tile BM x BN x 64, 256 threads = 4 waves in a 2x2 grid, each wave (BM/2)x(BN/2) as 32x32 MFMA
// tiles, double-buffered LDS, four k-steps of global loads in flight in registers.
#pragma once
#include "attn_decode_kernels.h"
#include "common.h"
#include <atomic>
#include <stdlib.h>

namespace fx {

constexpr int kGemmBK = 64;        // k-bytes per stage
// LDS tile layout: [16-byte k-chunk (4 per stage)][row][16 B], i.e. for one k-chunk the rows are contiguous.
// A wave-wide 128-bit fragment read then touches two contiguous 512-byte runs; the +32 B on the plane pitch
// spreads the four chunks of one row, written by four neighbouring lanes, over all banks.
__host__ __device__ constexpr int gemm_plane(int rows) { return rows * 16 + 32; }

enum GemmEpi { kGemmRaw = 0, kGemmDequant = 1, kGemmDequantAsym = 2 };

// 16 nibbles (8 bytes, low nibble = even index) -> 16 bytes in index order; SIGNED: two's-complement nibbles
// are sign-extended (the weights), otherwise they stay 0..15 (the activations).
template <bool SIGNED>
__device__ __forceinline__ i32x4 unpack16_nibbles(uint2 p) {
    i32x4 r;
    const uint32_t src[2] = {p.x, p.y};
#pragma unroll
    for (int h = 0; h < 2; h++) {
        uint32_t lo = src[h] & 0x0F0F0F0Fu, hi = (src[h] >> 4) & 0x0F0F0F0Fu;       // elements 0,2,4,6 and 1,3,5,7
        if constexpr (SIGNED) {
            lo |= (lo & 0x08080808u) * 30u;                                          // 0x08 -> 0xF8: sign bits of the byte
            hi |= (hi & 0x08080808u) * 30u;
        }
        r[2 * h] = (int)__builtin_amdgcn_perm(hi, lo, 0x05010400u);                 // bytes lo0, hi0, lo1, hi1
        r[2 * h + 1] = (int)__builtin_amdgcn_perm(hi, lo, 0x07030602u);             // bytes lo2, hi2, lo3, hi3
    }
    return r;
}

// PACKED: both operands hold two 4-bit values per byte (rows of k/2 bytes; activations unsigned, weights signed);
// they are widened to int8 between the global load and the LDS store, the MFMA path is the same.
template <int BM, int BN, int EPI, int D, bool PACKED = false>
__global__ __launch_bounds__(256) void gemm_i8_kernel(const int8_t* __restrict__ a, const int8_t* __restrict__ w,
                                                      int32_t* __restrict__ c_out, const float* __restrict__ s_x,
                                                      const float* __restrict__ w_s, const float* __restrict__ residual,
                                                      float* __restrict__ y, int m, int k, int n, int tiles_m, int tiles_n,
                                                      const float* __restrict__ b_x = nullptr, const float* __restrict__ w_sum = nullptr) {
    constexpr int WM = BM / 2, WN = BN / 2;          // wave tile
    constexpr int TM = WM / 32, TN = WN / 32;        // 32x32 MFMA tiles per wave
    constexpr int A_CHUNKS = BM * 4 / 256;           // 16-byte chunks per thread per stage
    constexpr int B_CHUNKS = BN * 4 / 256;
    constexpr int PA = gemm_plane(BM), PB = gemm_plane(BN);
    __shared__ __attribute__((aligned(16))) int8_t lds_a[2][4 * PA];
    __shared__ __attribute__((aligned(16))) int8_t lds_b[2][4 * PB];

    // XCD-aware tile order.  Consecutive workgroup ids land on different XCDs (8 of them, each with its own
    // 4 MiB L2).  Give every XCD a contiguous range of weight columns and walk the token-row tiles fastest,
    // so that a weight block is fetched from HBM by one XCD only and is shared there by all token-row tiles
    // (the activations, M x K, are small and are read by every XCD).
    int tm, tn;
    if ((tiles_n & 7) == 0) {
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        tn = xcd * (tiles_n >> 3) + idx / tiles_m;
        tm = idx % tiles_m;
    } else {
        tm = blockIdx.x / tiles_n;
        tn = blockIdx.x % tiles_n;
    }
    const int row0 = tm * BM, col0 = tn * BN;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;

    // global -> register staging: chunk id c = t + 256*i -> row c/4, 16-byte column c%4.  D k-steps of global
    // loads are kept in flight in registers (an L2/HBM round trip is several k-steps long).
    i32x4 ra[D][A_CHUNKS], rb[D][B_CHUNKS];
    const int8_t* a_ptr[A_CHUNKS];
    const int8_t* b_ptr[B_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) {
        const int c = t + 256 * i;
        a_ptr[i] = PACKED ? a + (size_t)min(row0 + (c >> 2), m - 1) * (k >> 1) + (c & 3) * 8
                          : a + (size_t)min(row0 + (c >> 2), m - 1) * k + (c & 3) * 16;
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
        const int c = t + 256 * i;
        b_ptr[i] = PACKED ? w + (size_t)min(col0 + (c >> 2), n - 1) * (k >> 1) + (c & 3) * 8
                          : w + (size_t)min(col0 + (c >> 2), n - 1) * k + (c & 3) * 16;
    }
    auto load_global = [&](int k0, i32x4 (&xa)[A_CHUNKS], i32x4 (&xb)[B_CHUNKS]) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) {
            if constexpr (PACKED) xa[i] = unpack16_nibbles<false>(*reinterpret_cast<const uint2*>(a_ptr[i] + (k0 >> 1)));
            else xa[i] = *reinterpret_cast<const i32x4*>(a_ptr[i] + k0);
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) {
            if constexpr (PACKED) xb[i] = unpack16_nibbles<true>(*reinterpret_cast<const uint2*>(b_ptr[i] + (k0 >> 1)));
            else xb[i] = *reinterpret_cast<const i32x4*>(b_ptr[i] + k0);
        }
    };
    auto store_lds = [&](int buf, const i32x4 (&xa)[A_CHUNKS], const i32x4 (&xb)[B_CHUNKS]) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) {
            const int c = t + 256 * i;
            *reinterpret_cast<i32x4*>(&lds_a[buf][(c & 3) * PA + (c >> 2) * 16]) = xa[i];
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) {
            const int c = t + 256 * i;
            *reinterpret_cast<i32x4*>(&lds_b[buf][(c & 3) * PB + (c >> 2) * 16]) = xb[i];
        }
    };

    i32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    const int nk = k / kGemmBK;            // a multiple of D (checked by the launcher)
#pragma unroll
    for (int d = 0; d < D; d++)
        if (d < nk) load_global(d * kGemmBK, ra[d], rb[d]);
    store_lds(0, ra[0], rb[0]);
    __syncthreads();
    const int frag_row = (lane & 31) * 16, frag_g = lane >> 5;
    for (int kt0 = 0; kt0 < nk; kt0 += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            const int kt = kt0 + d;
            const int buf = kt & 1;
            // slot d held k-step kt, which is already in LDS: refill it with k-step kt+D
            if (kt + D < nk) load_global((kt + D) * kGemmBK, ra[d], rb[d]);
#pragma unroll
            for (int ks = 0; ks < kGemmBK / 32; ks++) {
                i32x4 fa[TM], fb[TN];
#pragma unroll
                for (int i = 0; i < TM; i++)
                    fa[i] = *reinterpret_cast<const i32x4*>(&lds_a[buf][(ks * 2 + frag_g) * PA + (wm + i * 32) * 16 + frag_row]);
#pragma unroll
                for (int j = 0; j < TN; j++)
                    fb[j] = *reinterpret_cast<const i32x4*>(&lds_b[buf][(ks * 2 + frag_g) * PB + (wn + j * 32) * 16 + frag_row]);
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
            if (kt + 1 < nk) {
                store_lds(buf ^ 1, ra[(d + 1) % D], rb[(d + 1) % D]);   // the other buffer was last read before the previous barrier
                __syncthreads();
            }
        }
    }

    // epilogue: 32x32 accumulator layout - lane l holds column l%32, register r holds row 8*(r/4) + 4*(l/32) + r%4
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = col0 + wn + j * 32 + (lane & 31);
            if (col >= n) continue;
            float ws = 0.0f, wsm = 0.0f;
            if constexpr (EPI != kGemmRaw) ws = w_s[col];
            if constexpr (EPI == kGemmDequantAsym) wsm = w_sum[col];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = row0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                if (row >= m) continue;
                if constexpr (EPI != kGemmRaw) {
                    float v = (float)acc[i][j][r] * s_x[row] * ws;
                    if constexpr (EPI == kGemmDequantAsym) v = v + b_x[row] * wsm;      // zero point times the row sum of W
                    if (residual) v = v + residual[(size_t)row * n + col];
                    y[(size_t)row * n + col] = v;
                } else {
                    c_out[(size_t)row * n + col] = acc[i][j][r];
                }
            }
        }
}

// ---------------------------------------------------------------------------------------------------------
// Second kernel: tiles go global -> LDS by direct loads (global_load_lds_dwordx4), bypassing registers, two to four
// stages deep.  Tile BM x BN, BKB = 64 or 128 k-bytes per row and stage, four waves (2x2) or eight (2x4, or two
// k-groups of 2x2); the wave tile is a grid of 32x32 MFMA tiles, and the wider it is the more MFMAs every fragment
// read from LDS feeds (a 128x64 wave tile: six reads for eight MFMAs).
//
// LDS stage layout: row-major, BKB bytes (= BKB/16 16-byte k-chunks) per tile row.  A direct load writes lane i
// at base + 16*i, i.e. 64/(BKB/16) rows per instruction, which is also the coalesced order in global memory.  To
// keep the MFMA fragment reads (32 rows x one chunk) free of bank conflicts the chunks of a row are stored rotated:
// slot s of row r holds k-chunk s ^ ((r >> 2) & 3) for 64-byte rows, s ^ ((r >> 1) & 7) for 128-byte rows.  The
// rotation is applied on the global side of the direct load (the LDS side is fixed by the hardware).
//
// The loads are issued from inline assembly: the compiler does not track them, so the k-loop waits for them
// with explicit counters (results return in issue order).
__host__ __device__ constexpr int gemm_dma_lds_bytes(int bm, int bn, int stages, int bkb = 64, int nw = 4, int ksplit = 1) {
    // the stage rings (one per k-group), or the epilogue: one patch per wave plus, with two k-groups, the second
    // group's accumulators
    const int rings = ksplit * stages * (bm + bn) * bkb;
    const int epi = nw * 32 * 36 * 4 + (ksplit > 1 ? bm * bn * 4 : 0);
    return rings > epi ? rings : epi;
}

enum GemmDmaEpi { kDmaRaw = 0, kDmaDequant = 1, kDmaSwiglu = 2, kDmaQkv = 3, kDmaDequantAsym = 4, kDmaSwigluAsym = 5 };

// Arguments of the q/k/v epilogue: the 64-column tile of the fused [q | k | v] projection is one attention head,
// so RoPE (pairs k, k+32), the static int8 quantisation and the store into q8 / the K cache / the transposed V
// cache blocks all happen on the tile (64 tokens x 64 channels; a V cache block is 64 positions x 64 channels).
struct QkvEpiArgs {
    const float *sin_t = nullptr, *cos_t = nullptr, *q_s = nullptr, *k_s = nullptr, *v_s = nullptr;
    int8_t *q8 = nullptr, *kc = nullptr, *vc = nullptr;
    int pos0 = 0, q_heads = 0, kv_heads = 0, max_pos = 0;
    // asymmetric activations (kDmaDequantAsym / kDmaSwigluAsym; optional for kDmaQkv, null = symmetric): zero point per
    // row, weight row sum (times its scale) per column
    const float *b_x = nullptr, *w_sum = nullptr;
};

__device__ __forceinline__ void gemm_dma_issue(const int8_t* base, unsigned voff, unsigned lds_dst) {
    unsigned saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\t"
                 "s_mov_b32 m0, %3\n\t"
                 "s_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %2\n\t"
                 "s_mov_b32 m0, %0"
                 : "=&s"(saved_m0) : "v"(voff), "s"(base), "s"(lds_dst) : "memory");
}

template <int N>
__device__ __forceinline__ void gemm_wait_vmcnt() {            // s_waitcnt vmcnt(N) only; the count is a 6-bit split immediate
    static_assert(N >= 0 && N < 64, "vmcnt range");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// kDmaStages LDS stages; WPE = waves per SIMD the register allocation has to leave room for.
// BKB = k-bytes of a row per stage, 64 or 128.  A 64-byte segment is half a cache line, and the other half is asked
// for again one stage later: measured with the loads alone (no math, 128 x 256 tiles at K = 2048), the chip moves
// 23 TB/s into LDS in whole 128-byte lines and 14.5 TB/s in halves.  With 128-byte rows the slot rotation is
// s ^ ((r >> 1) & 7): two rows span the 64 banks, so 16 consecutive rows of one chunk fall on 16 different bank groups.
// NW = waves per workgroup, 4 (2x2 wave grid) or 8 (2x4): eight waves let a 256x256 tile keep two waves per SIMD.
// KSPLIT = 2 (with NW = 8): two groups of four waves work on the same output tile, group g on the stages
// kt with kt % 2 == g, each with its own ring of LDS stages; the second group's accumulators are added to the first's
// through LDS before the epilogue (integer sums: exact in any order).  For outputs too narrow to give every CU two
// workgroups (down projection: 256 tiles of 64x128) this puts two independent load pipelines on a CU all the same.
template <int BM, int BN, int EPI, int kDmaStages, int WPE, int BKB, int NW, int KSPLIT>   // at most 7 stages (the wait below distinguishes up to 5 younger ones)
__global__ __launch_bounds__(NW * 64, WPE) void gemm_i8_dma_kernel(const int8_t* __restrict__ a, const int8_t* __restrict__ w,
                                                          int32_t* __restrict__ c_out, const float* __restrict__ s_x,
                                                          const float* __restrict__ w_s, const float* __restrict__ residual,
                                                          float* __restrict__ y, int m, int k, int n, int tiles_m, int tiles_n,
                                                          QkvEpiArgs qa) {
    static_assert(NW == 4 || NW == 8, "four or eight waves");
    static_assert(KSPLIT == 1 || (KSPLIT == 2 && NW == 8 && EPI != kDmaQkv), "two k-groups need eight waves");
    constexpr int GW = NW / KSPLIT;                           // waves per k-group
    constexpr int WGN = GW / 2;                               // waves along N
    constexpr int WM = BM / 2, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    static_assert(BKB == 64 || BKB == 128, "64 or 128 k-bytes per row and stage");
    constexpr int CPR = BKB / 16, RPI = 64 / CPR;             // 16-byte chunks per row; rows per direct load (1 KiB)
    constexpr int A_INSTR = BM / (GW * RPI), B_INSTR = BN / (GW * RPI);   // direct loads per wave per stage
    static_assert(A_INSTR >= 1 && B_INSTR >= 1 && TM >= 1 && TN >= 1, "tile too small for this wave count");
    constexpr int STAGE = (BM + BN) * BKB, KS = BKB / 32;     // KS MFMA k-steps per stage
    auto rot = [](int r) { return BKB == 64 ? (r >> 2) & 3 : (r >> 1) & 7; };
    extern __shared__ __attribute__((aligned(16))) int8_t gemm_smem[];

    int tm, tn;
    if ((tiles_n & 7) == 0) {                                  // see gemm_i8_kernel: one range of weight columns per XCD
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        tn = xcd * (tiles_n >> 3) + idx / tiles_m;
        tm = idx % tiles_m;
    } else {
        tm = blockIdx.x / tiles_n;
        tn = blockIdx.x % tiles_n;
    }
    int row0 = tm * BM, col0 = tn * BN;
    const int t = threadIdx.x, lane = t & 63;
    const int wave_wg = __builtin_amdgcn_readfirstlane(t >> 6);
    const int grp = wave_wg / GW, wave = wave_wg % GW;         // k-group, wave within the group
    const int wm = (wave / WGN) * WM, wn = (wave % WGN) * WN;
    int8_t* const ring = gemm_smem + grp * (kDmaStages * STAGE);

    // per-lane global offsets of this wave's direct loads (without the k offset, which is uniform)
    unsigned offa[A_INSTR], offb[B_INSTR];
#pragma unroll
    for (int j = 0; j < A_INSTR; j++) {
        const int r = (wave * A_INSTR + j) * RPI + lane / CPR;
        offa[j] = (unsigned)min(row0 + r, m - 1) * (unsigned)k + (unsigned)(((lane % CPR) ^ rot(r)) * 16);
    }
#pragma unroll
    for (int j = 0; j < B_INSTR; j++) {
        const int r = (wave * B_INSTR + j) * RPI + lane / CPR;
        offb[j] = (unsigned)min(col0 + r, n - 1) * (unsigned)k + (unsigned)(((lane % CPR) ^ rot(r)) * 16);
    }
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)ring;
    // kt counts the stages of this k-group; the group's stage kt is stage kt * KSPLIT + grp of the whole K range
    auto issue_stage = [&](int kt) {
        const unsigned sb = lds0 + (unsigned)(kt % kDmaStages) * STAGE;
        const size_t koff = (size_t)(kt * KSPLIT + grp) * BKB;
#pragma unroll
        for (int j = 0; j < A_INSTR; j++) gemm_dma_issue(a + koff, offa[j], sb + (wave * A_INSTR + j) * 1024);
#pragma unroll
        for (int j = 0; j < B_INSTR; j++) gemm_dma_issue(w + koff, offb[j], sb + BM * BKB + (wave * B_INSTR + j) * 1024);
    };

    i32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    const int nk = k / (BKB * KSPLIT);                         // stages per k-group (the launcher checks divisibility)
    constexpr int PER = A_INSTR + B_INSTR;                     // direct loads per wave per stage
#pragma unroll
    for (int s0 = 0; s0 < kDmaStages - 1; s0++)
        if (s0 < nk) issue_stage(s0);
    // fragment addressing: lane l reads row (l % 32) of a 32-row tile, k-chunk 2*ks + l/32, from its rotated slot
    const int fr = lane & 31, fg = lane >> 5;
    auto read_frags = [&](int kt, int ks, i32x4 (&fa)[TM], i32x4 (&fb)[TN]) {
        const int8_t* sa = ring + (kt % kDmaStages) * STAGE;
        const int8_t* sb = sa + BM * BKB;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int r = wm + i * 32 + fr;
            fa[i] = *reinterpret_cast<const i32x4*>(sa + r * BKB + (((ks * 2 + fg) ^ rot(r)) * 16));
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int r = wn + j * 32 + fr;
            fb[j] = *reinterpret_cast<const i32x4*>(sb + r * BKB + (((ks * 2 + fg) ^ rot(r)) * 16));
        }
    };
    auto mma = [&](const i32x4 (&fa)[TM], const i32x4 (&fb)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };
    // stage kt has landed once only the younger stages in flight remain outstanding
    auto wait_stage = [&](int kt) {
        const int younger = min(kDmaStages - 2, nk - 1 - kt);
        if (younger >= 5) gemm_wait_vmcnt<(5 * PER < 64 ? 5 * PER : 63)>();
        else if (younger == 4) gemm_wait_vmcnt<(4 * PER < 64 ? 4 * PER : 63)>();
        else if (younger == 3) gemm_wait_vmcnt<3 * PER>();
        else if (younger == 2) gemm_wait_vmcnt<2 * PER>();
        else if (younger == 1) gemm_wait_vmcnt<PER>();
        else gemm_wait_vmcnt<0>();
    };

    // Software pipeline over k-steps of 32 bytes: the fragments of the next k-step are read from LDS before the
    // MFMAs of the current one are issued, so the LDS latency runs under matrix work.  The workgroup barrier
    // sits before the last k-step of a stage: after it stage kt+1 is complete in LDS and every wave has finished
    // reading stage kt, whose buffer the direct loads of the iteration after next overwrite.
    i32x4 fa0[TM], fb0[TN], fa1[TM], fb1[TN];
    wait_stage(0);
    __syncthreads();
    read_frags(0, 0, fa0, fb0);
    for (int kt = 0; kt < nk; kt++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks += 2) {
            read_frags(kt, ks + 1, fa1, fb1);
            if (ks == 0 && kt + kDmaStages - 1 < nk) issue_stage(kt + kDmaStages - 1);   // into the buffer that held stage kt-1
            __builtin_amdgcn_sched_barrier(0);
            mma(fa0, fb0);
            __builtin_amdgcn_sched_barrier(0);
            if (ks + 2 < KS) {
                read_frags(kt, ks + 2, fa0, fb0);
            } else if (kt + 1 < nk) {
                wait_stage(kt + 1);
                __syncthreads();
                read_frags(kt + 1, 0, fa0, fb0);
            }
            __builtin_amdgcn_sched_barrier(0);
            mma(fa1, fb1);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // Epilogue.  In the accumulator layout a lane holds ONE column (l%32) and 16 rows of a 32x32 tile, so direct
    // stores would be 4 bytes per lane.  Each wave instead turns its tiles through a private LDS patch
    // (32 x 36 words) and then owns 4 consecutive columns of a row: 16-byte loads of the residual, 16-byte stores
    // (8 bytes for the SiLU*up pairs), 128 contiguous bytes per row.
    __syncthreads();                                           // all waves are done with the stage buffers
    if constexpr (KSPLIT == 2) {
        // the second k-group hands its accumulators over, lane-contiguous (conflict-free), behind the patch area
        int* xch = reinterpret_cast<int*>(gemm_smem) + NW * 32 * 36 + wave * (TM * TN * 16 * 64) + lane;
        if (grp == 1) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) xch[((i * TN + j) * 16 + r) * 64] = acc[i][j][r];
        }
        __syncthreads();
        if (grp == 1) return;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] += xch[((i * TN + j) * 16 + r) * 64];
    }
    if constexpr (EPI == kDmaQkv) {
        static_assert(EPI != kDmaQkv || (BM == 64 && BN == 64 && NW == 4), "the q/k/v epilogue works on 64x64 tiles with four waves");
        constexpr int TP = 65;                                 // odd pitch: a column walk hits every bank once
        float* tile = reinterpret_cast<float*>(gemm_smem);     // dequantised tile [64 tokens][64 channels]
        {
            const int col = col0 + wn + (lane & 31);
            const float ws = w_s[col];
            const bool asym = qa.b_x != nullptr;              // asymmetric activations: + zero point x row sum of the dequantised weights
            const float wq = asym ? qa.w_sum[col] : 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int lr = wm + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                const int row = min(row0 + lr, m - 1);
                float v = (float)acc[0][0][r] * s_x[row] * ws;
                if (asym) v = v + qa.b_x[row] * wq;
                tile[lr * TP + wn + (lane & 31)] = v;
            }
        }
        __syncthreads();
        const int head = col0 / kHd;                           // uniform: 0..q_heads-1 q, then k heads, then v heads
        const int sel = t & 63, part = t >> 6;
        if (head < qa.q_heads + qa.kv_heads) {
            // RoPE + static quantisation: thread = (token sel, pairs 8*part .. 8*part+7)
            const int row = row0 + sel, pos = qa.pos0 + row;
            if (row < m) {
                const bool is_q = head < qa.q_heads;
                const int hk = is_q ? head : head - qa.q_heads;
                const float div = is_q ? 8.0f * qa.q_s[hk] : 1.0f * qa.k_s[hk];     // sqrt(head_dim) folded into the Q scale
                const float* sn = qa.sin_t + (size_t)pos * 32 + part * 8;
                const float* cs = qa.cos_t + (size_t)pos * 32 + part * 8;
                uint32_t lo[2] = {0, 0}, hi[2] = {0, 0};
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float t0 = tile[sel * TP + part * 8 + j], t1 = tile[sel * TP + part * 8 + j + 32];
                    const float o0 = t0 * cs[j] - t1 * sn[j];
                    const float o1 = t0 * sn[j] + t1 * cs[j];
                    lo[j >> 2] |= (uint32_t)(static_q8(o0, div) & 0xff) << (8 * (j & 3));
                    hi[j >> 2] |= (uint32_t)(static_q8(o1, div) & 0xff) << (8 * (j & 3));
                }
                int8_t* dst = is_q ? qa.q8 + ((size_t)row * qa.q_heads + hk) * kHd : qa.kc + k_index(hk, pos, qa.max_pos);
                *reinterpret_cast<uint2*>(dst + part * 8) = make_uint2(lo[0], lo[1]);
                *reinterpret_cast<uint2*>(dst + part * 8 + 32) = make_uint2(hi[0], hi[1]);
            }
        } else {
            // V: thread = (channel sel, 16 consecutive positions 16*part ..): one 16-byte run of the transposed cache block
            const int hv = head - qa.q_heads - qa.kv_heads;
            const int rbase = row0 + part * 16;
            if (rbase < m) {                                   // m is a multiple of 32 (checked by the launcher)
                const float div = 1.0f * qa.v_s[hv];
                uint32_t wv4[4] = {0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < 16; i++)
                    wv4[i >> 2] |= (uint32_t)(static_q8(tile[(part * 16 + i) * TP + sel], div) & 0xff) << (8 * (i & 3));
                *reinterpret_cast<uint4*>(qa.vc + v_index(hv, qa.pos0 + rbase, sel, qa.max_pos)) = make_uint4(wv4[0], wv4[1], wv4[2], wv4[3]);
            }
        }
        return;
    }
    constexpr bool kAsym = EPI == kDmaDequantAsym || EPI == kDmaSwigluAsym;      // + zero point x row sum of the dequantised weights
    constexpr bool kPlain = EPI == kDmaDequant || EPI == kDmaDequantAsym;        // fp32 outputs (+ residual); else SiLU(gate) * up pairs
    constexpr int EP = 36;                                     // patch pitch in words (rows stay 16-byte aligned)
    int* patch = reinterpret_cast<int*>(gemm_smem) + wave * (32 * EP);
    const int pr = lane >> 3, pc = (lane & 7) * 4;             // row within a group of 8, first of this lane's 4 columns
    // Every scale this lane needs is loaded before the first tile: a load inside the tile loop would be waited for
    // together with the stores issued before it (one counter covers both), once per group of rows.
    float sxv[TM][4];
    float4 wsv[TN];
    float bxv[kAsym ? TM : 1][4];
    float4 wsumv[kAsym ? TN : 1];
    if constexpr (EPI != kDmaRaw) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int p = 0; p < 4; p++) sxv[i][p] = s_x[min(row0 + wm + i * 32 + p * 8 + pr, m - 1)];
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = col0 + wn + j * 32 + pc;
            wsv[j] = col < n ? *reinterpret_cast<const float4*>(w_s + col) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    }
    if constexpr (kAsym) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int p = 0; p < 4; p++) bxv[i][p] = qa.b_x[min(row0 + wm + i * 32 + p * 8 + pr, m - 1)];
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = col0 + wn + j * 32 + pc;
            wsumv[j] = col < n ? *reinterpret_cast<const float4*>(qa.w_sum + col) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int col = col0 + wn + j * 32 + pc;               // n is a multiple of 4 (checked by the launcher)
        const bool col_ok = col < n;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            float4 rs[4];                                      // the tile's residual rows, in flight during the turn through LDS
            bool has_res = false;
            if constexpr (kPlain) {
                has_res = residual != nullptr;
                if (has_res) {
#pragma unroll
                    for (int p = 0; p < 4; p++) {
                        const int row = row0 + wm + i * 32 + p * 8 + pr;
                        rs[p] = col_ok && row < m ? *reinterpret_cast<const float4*>(residual + (size_t)row * n + col)
                                                  : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 16; r++)
                patch[((r >> 2) * 8 + (lane >> 5) * 4 + (r & 3)) * EP + (lane & 31)] = acc[i][j][r];
            // the patch is private to the wave: the LDS operations of a wave complete in order, the compiler is kept from
            // moving them across this point
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // One explicit wait per tile, outside the guarded stores: the scales (first tile) and this tile's residual
            // rows have landed.  Left to the compiler the wait sits behind the store guards, is repeated for every group
            // of rows, and then also waits for the store issued just before it.
            if constexpr (EPI != kDmaRaw) { if ((i == 0 && j == 0) || has_res) gemm_wait_vmcnt<0>(); }
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const int lr = p * 8 + pr;
                const int row = row0 + wm + i * 32 + lr;
                const i32x4 v = *reinterpret_cast<const i32x4*>(patch + lr * EP + pc);
                // the arithmetic runs for every lane and only the store is guarded: a wait placed behind a branch
                // would be repeated at every later use, and there it would also wait for the stores in between
                const bool ok = col_ok && row < m;
                if constexpr (EPI == kDmaRaw) {
                    if (ok) *reinterpret_cast<i32x4*>(c_out + (size_t)row * n + col) = v;
                } else {
                    const float sx = sxv[i][p];
                    const float4 ws = wsv[j];
                    float4 o;
                    o.x = (float)v[0] * sx * ws.x; o.y = (float)v[1] * sx * ws.y;
                    o.z = (float)v[2] * sx * ws.z; o.w = (float)v[3] * sx * ws.w;
                    if constexpr (kAsym) {
                        const float bx = bxv[i][p];
                        const float4 wq = wsumv[j];
                        o.x = o.x + bx * wq.x; o.y = o.y + bx * wq.y; o.z = o.z + bx * wq.z; o.w = o.w + bx * wq.w;
                    }
                    if constexpr (kPlain) {
                        if (has_res) { o.x = o.x + rs[p].x; o.y = o.y + rs[p].y; o.z = o.z + rs[p].z; o.w = o.w + rs[p].w; }
                        if (ok) *reinterpret_cast<float4*>(y + (size_t)row * n + col) = o;
                    } else {
                        // weight rows are interleaved (2c gate, 2c+1 up): columns (col, col+1) and (col+2, col+3) are pairs
                        float2 h;
                        h.x = o.y * silu_f(o.x);
                        h.y = o.w * silu_f(o.z);
                        if (ok) *reinterpret_cast<float2*>(y + (size_t)row * (n >> 1) + (col >> 1)) = h;
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();               // reads of this tile before the next tile's writes
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
}

template <int BM, int BN, int EPI, int STAGES = 3, int WPE = 1, int BKB = 64, int NW = 4, int KSPLIT = 1>
inline int launch_gemm_dma(const int8_t* a, const int8_t* w, int32_t* c, const float* s_x, const float* w_s,
                           const float* residual, float* y, int m, int k, int n, hipStream_t st, QkvEpiArgs qa = QkvEpiArgs()) {
    static std::atomic<bool> opted_in{false};             // more than the default 64 KiB of LDS per workgroup
    if (!opted_in.load(std::memory_order_acquire)) {   // idempotent: two threads racing here both set the same attribute
        FX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_i8_dma_kernel<BM, BN, EPI, STAGES, WPE, BKB, NW, KSPLIT>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, gemm_dma_lds_bytes(BM, BN, STAGES, BKB, NW, KSPLIT)));
        opted_in.store(true, std::memory_order_release);
    }
    const int tm = (m + BM - 1) / BM, tn = (n + BN - 1) / BN;
    gemm_i8_dma_kernel<BM, BN, EPI, STAGES, WPE, BKB, NW, KSPLIT><<<tm * tn, NW * 64, gemm_dma_lds_bytes(BM, BN, STAGES, BKB, NW, KSPLIT), st>>>(a, w, c, s_x, w_s, residual, y, m, k, n, tm, tn, qa);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

template <int EPI>
inline int launch_gemm(const int8_t* a, const int8_t* w, int32_t* c, const float* s_x, const float* w_s,
                       const float* residual, float* y, int m, int k, int n, hipStream_t st) {
    // Measured on MI355X at M=1024: the direct-load kernel wins wherever it applies; 128x128 tiles once they fill
    // the chip about three times over, 64x64 tiles for the narrow projections.  FLEXLLM_GEMM_TILE forces a variant
    // (0..2: register-staged 128x128 / 64x128 / 64x64; direct-load: 11 = 128x128, 12 = 128x128 with two stages of
    // 128-byte rows, 13 = 64x64, 19 = 64x128 four
    // stages, all with 64-byte rows; 36 = 64x64 four stages and 38 = 64x64 three stages with 128-byte rows; 60 = 64x128
    // three stages with 128-byte rows and two k-groups).
    auto tiles = [&](int bm, int bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    static const char* force = getenv("FLEXLLM_GEMM_TILE");
    // the direct-load kernel needs 32-bit element offsets into both operands and 16-byte aligned output rows
    const bool dma_ok = (size_t)m * k < (1ull << 31) && (size_t)n * k < (1ull << 31) && n % 4 == 0;
    int mode = dma_ok ? (tiles(128, 128) >= 768 ? 11 : (k >= 4096 && tiles(64, 128) >= 256) ? 19 : 13) : (tiles(128, 128) >= 1024 ? 0 : 2);
    // whole 128-byte lines per row and stage where K allows: three workgroups of 48 KiB per CU when the grid has
    // that many, else two of 64 KiB with a fourth stage (the narrow projections stream their weights cold)
    // Long K and an output too narrow for two workgroups per CU (down projection): 64x128 tiles, two k-groups of
    // four waves per workgroup (32 us against 36 us for 64x64 tiles, two workgroups per CU).
    // 384..767 tiles of 128x128 (o and down projections from M = 3072): two stages of 128-byte rows, two workgroups
    // per CU.  At M = 4096: 36 us against 47 us (o) and 102 us against 133 us (down) for the narrow-tile choices below;
    // at M = 3072: 30 / 87 us against 35 / 109 us; at M = 2048 (256 tiles) the narrow tiles are level or ahead.
    if (dma_ok && mode != 11 && k % 128 == 0 && tiles(128, 128) >= 384) mode = 12;
    if (mode == 19 && k % 256 == 0) mode = 60;
    if ((mode == 13 || mode == 19) && k % 128 == 0) mode = tiles(64, 64) >= 768 ? 38 : 36;
    if (force) mode = atoi(force);
    if (mode >= 10 && !dma_ok) mode = 2;
    const int nk = k / kGemmBK;
    if (mode >= 10) {
        constexpr int DE = EPI == kGemmDequant ? kDmaDequant : kDmaRaw;
        if (mode == 12 && k % 128 == 0) return launch_gemm_dma<128, 128, DE, 2, 2, 128>(a, w, c, s_x, w_s, residual, y, m, k, n, st);
        if (mode == 11) return launch_gemm_dma<128, 128, DE>(a, w, c, s_x, w_s, residual, y, m, k, n, st);
        if (mode == 19) return launch_gemm_dma<64, 128, DE, 4, 2>(a, w, c, s_x, w_s, residual, y, m, k, n, st);
        if (k % 128 == 0) {
            if (mode == 36) return launch_gemm_dma<64, 64, DE, 4, 2, 128>(a, w, c, s_x, w_s, residual, y, m, k, n, st);
            if (mode == 38) return launch_gemm_dma<64, 64, DE, 3, 3, 128>(a, w, c, s_x, w_s, residual, y, m, k, n, st);
            if (k % 256 == 0) {
                if (mode == 60) return launch_gemm_dma<64, 128, DE, 3, 2, 128, 8, 2>(a, w, c, s_x, w_s, residual, y, m, k, n, st);
            }
        }
        return launch_gemm_dma<64, 64, DE>(a, w, c, s_x, w_s, residual, y, m, k, n, st);
    }
#define FX_GEMM_LAUNCH(BM, BN, DD)                                                                                \
    do {                                                                                                          \
        const int tm = (m + BM - 1) / BM, tn = (n + BN - 1) / BN;                                                 \
        gemm_i8_kernel<BM, BN, EPI, DD><<<tm * tn, 256, 0, st>>>(a, w, c, s_x, w_s, residual, y, m, k, n, tm, tn); \
    } while (0)
    const bool deep = nk % 4 == 0;      // prefetch depth 4 needs the k-steps in groups of 4 (K % 256 == 0)
    if (mode == 0) { if (deep) FX_GEMM_LAUNCH(128, 128, 4); else FX_GEMM_LAUNCH(128, 128, 1); }
    else if (mode == 1) { if (deep) FX_GEMM_LAUNCH(64, 128, 4); else FX_GEMM_LAUNCH(64, 128, 1); }
    else { if (deep) FX_GEMM_LAUNCH(64, 64, 4); else FX_GEMM_LAUNCH(64, 64, 1); }
#undef FX_GEMM_LAUNCH
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

// Asymmetric activations held one value per byte (0..127, e.g. the uint4 values of the W4A4 path before packing) times
// int8 weights on the direct-load kernel: y = (float(acc) * s_x) * w_s + b_x * w_sum (+ residual).
inline int launch_gemm_asym(const int8_t* a, const int8_t* w, const float* s_x, const float* b_x, const float* w_s,
                            const float* w_sum, const float* residual, float* y, int m, int k, int n, hipStream_t st) {
    FX_REQUIRE((size_t)m * k < (1ull << 31) && (size_t)n * k < (1ull << 31) && n % 4 == 0,
               "linear_i8_gemm_dequant_asym: m=%d k=%d n=%d outside the direct-load kernel's range", m, k, n);
    auto tiles = [&](int bm, int bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    QkvEpiArgs qa = QkvEpiArgs();
    qa.b_x = b_x; qa.w_sum = w_sum;
    constexpr int DE = kDmaDequantAsym;
    static const char* force = getenv("FLEXLLM_GEMM_TILE");
    const int fm = force ? atoi(force) : 0;
    // Wide outputs (the separate gate and up projections of the W4A4 graph, 2048 -> 8192 at M = 1024), measured (us):
    // 128x128 tiles, two stages of 128-byte rows 26.7; 128x128, three stages of 64-byte rows 31.8; 128x256 on four
    // waves 38.7; 64x64 tiles 41.0.
    if (k % 128 == 0 && (fm == 12 || (!fm && tiles(128, 128) >= 384)))
        return launch_gemm_dma<128, 128, DE, 2, 2, 128>(a, w, nullptr, s_x, w_s, residual, y, m, k, n, st, qa);
    if (fm == 11 || (!fm && tiles(128, 128) >= 768)) return launch_gemm_dma<128, 128, DE>(a, w, nullptr, s_x, w_s, residual, y, m, k, n, st, qa);
    if (k % 256 == 0 && k >= 4096 && tiles(64, 128) >= 256 && (!fm || fm == 60))
        return launch_gemm_dma<64, 128, DE, 3, 2, 128, 8, 2>(a, w, nullptr, s_x, w_s, residual, y, m, k, n, st, qa);
    if (k % 128 == 0) {
        if (tiles(64, 64) >= 768) return launch_gemm_dma<64, 64, DE, 3, 3, 128>(a, w, nullptr, s_x, w_s, residual, y, m, k, n, st, qa);
        return launch_gemm_dma<64, 64, DE, 4, 2, 128>(a, w, nullptr, s_x, w_s, residual, y, m, k, n, st, qa);
    }
    return launch_gemm_dma<64, 64, DE>(a, w, nullptr, s_x, w_s, residual, y, m, k, n, st, qa);
}

// The gate/up projection of the W4A4 graph (interleaved rows, asymmetric activations held one value per byte) with
// SiLU(gate)*up in the epilogue: the asymmetric dequantisation of launch_gemm_asym followed by the product that the
// Hadamard kernel would otherwise form from the interleaved fp32 columns - the same arithmetic, half the output.
// Tiles as in launch_gemm_swiglu: 256x256 where its grid fills the CUs in whole rounds (1024 tokens: 44 us against
// 50 us for the unfused 128x128 kernel, and the transform after it reads half as much), smaller ones otherwise.
inline int launch_gemm_swiglu_asym(const int8_t* a, const int8_t* w_gu, const float* s_x, const float* b_x, const float* w_s_gu,
                                   const float* w_sum_gu, float* h, int m, int k, int n2, hipStream_t st) {
    FX_REQUIRE((size_t)m * k < (1ull << 31) && (size_t)n2 * k < (1ull << 31) && n2 % 4 == 0,
               "linear_i8_gemm_swiglu_asym: m=%d k=%d n=%d outside the direct-load kernel's range", m, k, n2 / 2);
    auto tiles = [&](int bm, int bn) { return ((m + bm - 1) / bm) * ((n2 + bn - 1) / bn); };
    QkvEpiArgs qa = QkvEpiArgs();
    qa.b_x = b_x; qa.w_sum = w_sum_gu;
    constexpr int E = kDmaSwigluAsym;
    if (k % 128 == 0) {
        const int t256 = tiles(256, 256);
        if (t256 >= 256 && (t256 % 256 == 0 || t256 >= 1024))
            return launch_gemm_dma<256, 256, E, 2, 2, 128, 8>(a, w_gu, nullptr, s_x, w_s_gu, nullptr, h, m, k, n2, st, qa);
        if (tiles(128, 128) >= 384) return launch_gemm_dma<128, 128, E, 2, 2, 128>(a, w_gu, nullptr, s_x, w_s_gu, nullptr, h, m, k, n2, st, qa);
        return launch_gemm_dma<64, 64, E, 4, 2, 128>(a, w_gu, nullptr, s_x, w_s_gu, nullptr, h, m, k, n2, st, qa);
    }
    return launch_gemm_dma<64, 64, E>(a, w_gu, nullptr, s_x, w_s_gu, nullptr, h, m, k, n2, st, qa);
}

// W4A4 prefill GEMM on nibble-packed operands (register-staged kernel, nibbles widened on the way to LDS).
template <int EPI>
inline int launch_gemm_u4i4(const uint8_t* a4, const uint8_t* w4, int32_t* c, const float* s_x, const float* b_x,
                            const float* w_s, const float* w_sum, const float* residual, float* y, int m, int k, int n, hipStream_t st) {
    const int8_t* a = reinterpret_cast<const int8_t*>(a4);
    const int8_t* w = reinterpret_cast<const int8_t*>(w4);
    const bool big = ((m + 127) / 128) * ((n + 127) / 128) >= 768;
    if (big) {
        const int tm = (m + 127) / 128, tn = (n + 127) / 128;
        gemm_i8_kernel<128, 128, EPI, 1, true><<<tm * tn, 256, 0, st>>>(a, w, c, s_x, w_s, residual, y, m, k, n, tm, tn, b_x, w_sum);
    } else {
        const int tm = (m + 63) / 64, tn = (n + 63) / 64;
        gemm_i8_kernel<64, 64, EPI, 1, true><<<tm * tn, 256, 0, st>>>(a, w, c, s_x, w_s, residual, y, m, k, n, tm, tn, b_x, w_sum);
    }
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

// Gate/up projection with the SiLU(gate)*up product in the epilogue; n2 = 2 * intermediate size (interleaved rows).
inline int launch_gemm_swiglu(const int8_t* a, const int8_t* w_gu, const float* s_x, const float* w_s_gu, float* h, int m,
                              int k, int n2, hipStream_t st) {
    FX_REQUIRE((size_t)m * k < (1ull << 31) && (size_t)n2 * k < (1ull << 31) && n2 % 4 == 0,
               "linear_i8_gemm_swiglu: m=%d k=%d n=%d outside the direct-load kernel's range", m, k, n2 / 2);
    // Measured at M=1024, 2048 -> 2x8192 (us): 256x256 tiles on eight waves, two stages of 128-byte rows, one
    // workgroup per CU: 42.0; the same with four stages of 64-byte rows: 43.6; 128x256 tiles on four waves, two
    // stages of 64-byte rows, two workgroups per CU: 49.3; 128x256 on eight waves: 48-57; 128x128 tiles (two or
    // three per CU) and 256x256 on four waves: 48-58.  The big tile is taken when its grid fills the 256 CUs in
    // whole rounds (or many of them); FLEXLLM_GEMM_TILE forces 50 / 16 / 13 (the 64x64 fallback).
    static const char* force = getenv("FLEXLLM_GEMM_TILE");
    const int tiles_256 = ((m + 255) / 256) * ((n2 + 255) / 256);
    const int tiles_big = ((m + 127) / 128) * ((n2 + 255) / 256);
    int mode = (k % 128 == 0 && tiles_256 >= 256 && (tiles_256 % 256 == 0 || tiles_256 >= 1024)) ? 50 : tiles_big >= 384 ? 16 : 13;
    if (force) mode = atoi(force);
    if (mode == 50 && k % 128 == 0)
        return launch_gemm_dma<256, 256, kDmaSwiglu, 2, 2, 128, 8>(a, w_gu, nullptr, s_x, w_s_gu, nullptr, h, m, k, n2, st);
    if (mode == 16) return launch_gemm_dma<128, 256, kDmaSwiglu, 2, 2>(a, w_gu, nullptr, s_x, w_s_gu, nullptr, h, m, k, n2, st);
    return launch_gemm_dma<64, 64, kDmaSwiglu>(a, w_gu, nullptr, s_x, w_s_gu, nullptr, h, m, k, n2, st);
}

// Fused q/k/v projection: GEMM over the concatenated [q | k | v] weight rows with RoPE, static int8 quantisation and
// the stores into q8 [tokens][q_heads][64], the K cache and the V cache in the epilogue.  Token i sits at position
// pos0 + i; pos0 % 64 == 0 and m % 32 == 0 so that a tile of 64 tokens is one block of the transposed V cache.
inline int launch_gemm_qkv(const int8_t* a, const int8_t* w_qkv, const float* s_x, const float* w_s, int m, int k,
                           const QkvEpiArgs& qa, hipStream_t st) {
    const int n = (qa.q_heads + 2 * qa.kv_heads) * kHd;
    FX_REQUIRE(m % 32 == 0 && qa.pos0 % 64 == 0 && qa.pos0 + m <= qa.max_pos, "gemm_qkv: m=%d pos0=%d max_pos=%d", m, qa.pos0, qa.max_pos);
    FX_REQUIRE((size_t)m * k < (1ull << 31) && (size_t)n * k < (1ull << 31), "gemm_qkv: m=%d k=%d outside the direct-load kernel's range", m, k);
    static const char* force = getenv("FLEXLLM_GEMM_TILE");
    const int mode = force ? atoi(force) : (((m + 63) / 64) * (n / 64) >= 768 ? 38 : 36);
    if (k % 128 == 0) {
        if (mode == 36) return launch_gemm_dma<64, 64, kDmaQkv, 4, 2, 128>(a, w_qkv, nullptr, s_x, w_s, nullptr, nullptr, m, k, n, st, qa);
        if (mode == 38) return launch_gemm_dma<64, 64, kDmaQkv, 3, 3, 128>(a, w_qkv, nullptr, s_x, w_s, nullptr, nullptr, m, k, n, st, qa);
    }
    return launch_gemm_dma<64, 64, kDmaQkv>(a, w_qkv, nullptr, s_x, w_s, nullptr, nullptr, m, k, n, st, qa);
}

}  // namespace fx

// One persistent kernel per decoded token: all 16 layers, the final norm and the output head (fp16 tied embedding for
// the W8A8 model, int4 head for the W4A4 model: the kernel body is a template over the precision).
//
// Why: at batch 1 a decode step is ~100 dependent phases of 0.3-4 us of HBM streaming each; as separate
// kernels every phase pays a launch plus a cold start, and the chip idles between them.  Here 256 workgroups
// (one per CU, 512 threads) stay resident and walk the phases together:
//   per layer  1 RMSNorm+quant (redundantly in every workgroup) -> q/k/v GEMV rows
//              2 RoPE + static int8 quant + KV append, int8 scores of a 128-key chunk, chunk max / sum-exp
//              3 row statistics from the chunk statistics, uint8 probabilities, partial P.V (int32 atomics)
//              4 attention dequant + per-token quant (redundant) -> o_proj rows + residual
//              5 RMSNorm+quant (redundant) -> gate/up rows + SiLU*up
//              6 Hadamard R4 + quant (redundant) -> down rows + residual
//   then       final RMSNorm (redundant) -> head rows, per-workgroup argmax candidates.
// Hand-overs between workgroups, by what measured fastest for each:
//   1->2, 2->3  few consumers (a KV head's 32 workgroups need 384 of the 3072 q/k/v outputs, then each other's chunk
//               statistics): each value is one 64-bit word with the sequence number of the layer pass in its high
//               half, and the consumers poll the words they need.
//   4->5, 6->1  the residual stream, which every workgroup needs in full: tagged words as well (2048 words polled by
//               every workgroup, each wave 256 of them in whole lines; a lane that has its values stops loading).
//               Faster than a grid barrier plus a load.  A wave's poll says that 32 producers have published;
//               "everybody has" holds for the workgroup only behind the workgroup barrier that follows the polls.
//   3->4        int32 atomic adds into the attention accumulators, then a grid barrier (device-scope relaxed atomics:
//               eight group counters, the last arriver of a group sets the group's release flag, everybody polls
//               the eight flags), then coherent loads.
//   5->6        SiLU(gate)*up (8192 floats): coherent stores into a slice that no other layer pass of the launch uses,
//               a grid barrier, then ORDINARY loads, which the 32 CUs of an XCD share through L2 (see MegaParams::h).
// The tagged arrays and the barrier's words exist once per I/O die, in memory attached to that die (MegaParams::xblk):
// producers store into both copies, consumers poll their own die's.
// A tagged slot is rewritten a layer later, after at least one exchange that all its readers take part in as
// producers, i.e. after they have finished with it.  The weights a workgroup needs in the NEXT phase do not depend on
// the activations, so they are requested BEFORE waiting: HBM keeps streaming while the hand-over is in flight.
//
// Wave roles.  Vector-memory results return to a wave in issue order, so a wave with a long weight prefetch in
// flight cannot see an activation load (or have a store acknowledged) until the prefetch has landed.  The
// two big matrices are therefore owned by waves 4..7 ("stream waves"): they issue the gate/up rows a full
// phase ahead and the down rows before the gate/up barrier, one slice per phase, each right after the phase's
// activation loads have landed.  Waves 0..3 own the small q/k/v and o_proj rows and do the global stores; only they
// drain their memory counter before arriving at a barrier.
//
// Memory-model discipline: every value that crosses workgroups inside a launch (x, x2, qkv, chunk statistics,
// attention accumulators, h) is written with device-scope relaxed atomic stores/adds, which are performed at the
// memory side (past the per-XCD L2), and - h apart - read with device-scope relaxed atomic loads; each thread drains
// its outstanding stores (s_waitcnt vmcnt(0)) before its workgroup arrives at a barrier.  There is one fence: a
// device-scope acquire at kernel start, which empties the XCD's L2 of clean lines so that h's ordinary loads cannot
// hit a line of an earlier launch.  Weights and the old KV cache are read-only inside a step and use ordinary
// loads; the new token's K/V row is used from LDS by the workgroup that owns its chunk and written to the cache for
// later steps (that workgroup is also the only one that reads it back within the launch).
// Every spin is bounded: on a time-out the kernel sets an error flag, every other wait sees the flag within 64
// polls, and the launch ends after the current token.
#pragma once
#include "attn_decode_kernels.h"
#include "gemv_i8.h"
#include "linear_w4a4.h"
#include "logits_kernels.h"
#include "prefill.h"
#include <hip/hip_fp16.h>

namespace fx {

constexpr int kMegaWG = 256;       // workgroups (persistent, one per CU)
constexpr int kMegaT = 512;        // threads per workgroup
constexpr int kMegaWaves = kMegaT / 64;
constexpr int kMegaGroup = 32;     // workgroups per first-level barrier counter
constexpr int kMegaGroups = kMegaWG / kMegaGroup;   // 8 first-level groups: workgroup w belongs to group w mod 8, the XCD it runs on
constexpr int kMegaFlagCopies = 8; // copies of each of the barrier's release flags: workgroup w polls copy w mod 8
constexpr int kMegaFlagBase = 64 * kMegaGroups;     // the flags follow the counters (in 32-bit words); flag (group g, copy r) at + 16 * (8 r + g)
constexpr int kMegaBarWords = kMegaFlagBase + 16 * kMegaFlagCopies * kMegaGroups;   // per die: 6 KiB
constexpr int kMegaSpinLimit = 1 << 20;   // polls of ~1 us each: a wait that has not ended after a second never will
constexpr int kMegaErrPeriod = 64;         // a spinning thread looks at the error flag every so many polls
constexpr int kMegaMaxSteps = 64;  // tokens per launch in greedy mode (bounds the run time of one launch)

struct MegaParams {
    const void* layers;            // device array [layers] of LayerW (W8A8) or LayerW4 (W4A4)
    const uint8_t* head_w4;        // W4A4: int4 output head, nibble-packed [vocab][hidden/2], with per-row scale and row sum
    const float *head_s, *head_sum;
    const float *gamma, *q_s, *k_s, *v_s, *a_s, *rope_sin, *rope_cos;
    const __half* embed;
    int8_t *k_cache, *v_cache;
    size_t cache_layer_bytes;
    float *x, *x2, *qkv, *logits;
    // SiLU(gate)*up after the workgroup-local Hadamard stages: [kMegaMaxSteps * layers][8192], one slice per layer pass
    // of a launch.  Every workgroup reads all of it, and with coherent (L2-bypassing) loads the 32 CUs of an XCD would
    // each pull the 32 KiB through the XCD's fabric port.  Because no address is written twice within a launch, and L2
    // holds nothing from before the launch (every workgroup starts with an acquire fence at device scope, which
    // drops the clean lines of its XCD's L2: lines of an earlier launch do survive a kernel boundary otherwise),
    // an ordinary load can never see a stale line: the first CU of an XCD to touch a line (after the barrier that
    // follows its write-through store) fetches it, the others hit in L2.
    float* h;
    float2* stats;                 // [q_heads][32] (one-kernel-per-stage path)
    // The words that cross workgroups inside a launch live in 8 KiB blocks of one arena, every array once per I/O die:
    // copy d is in memory attached to die d and is READ by the workgroups of that die's XCDs, while producers store
    // into both copies (a hand-over through the other die's memory takes 0.2-0.7 us longer).  Byte k of
    // xblk[d][k / 8] is the arena block that holds block k of die d's copy (kXb* below); when the placement of memory is
    // not known both dies name the same blocks.  Tagged arrays start as 0xFF..FF, accumulators and the barrier as 0.
    //   qkv    [H + 2 KV] tagged words = 3 blocks: q/k/v projection outputs, each with the layer pass's sequence number in its high word
    //   stats  [q_heads][2][32] tagged words = 2 blocks of 16 heads: chunk maxima, then chunk sums of exponentials
    //   x      [H] tagged words = 2 blocks: the residual stream after a layer (down projection + residual)
    //   x2     [H] tagged words = 2 blocks: the residual stream after attention (o projection + residual)
    //   o_acc  [H] int32 = 1 block: attention accumulators (zero at launch, cleared again once read).  One copy only (die 0's entry):
    //          adding every part twice costs more than the reads across the dies (measured)
    //   bar    1 block: grid barrier, see GridBarrier
    char* xarena;
    unsigned long long xblk[2][2];
    unsigned die_mask;             // bit x = the I/O die of XCD x
    int* state;                    // [0] pos, [1] step, [2] barrier epoch base, [3] error flag, [4] layer sequence number base
    int* token;                    // current token id (device), used when x_in == NULL; greedy mode leaves the last token here
    int* tokens_out;               // greedy mode: generated ids are written to tokens_out[state[1] + step]; NULL otherwise
    int n_steps;                   // tokens per launch (> 1 only in greedy mode)
    const float* x_in;             // optional fp32 input embedding
    float* am_v;                   // [kMegaWG] argmax candidates
    int* am_i;
    // top-k sampling instead of arg-max (top_k > 0): step s draws with rands[state[1] + s]; per-workgroup candidates
    int top_k;
    const float* rands;
    float* cand_v;                 // [kMegaWG][kTopKMax]
    int* cand_i;
    int n_layers, max_pos, vocab, want_head;
    float eps, fht_scale;
    int timeline_wg;               // the workgroup whose stamps the timeline holds
    long long* timeline;           // optional [n_layers*6+2][2] wall-clock stamps of workgroup 0 (after wait, before arrive)
};

__device__ __forceinline__ float ld_f(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// Two / four consecutive floats with 64-bit coherent loads (p 8-byte aligned): half the vector-memory instructions
// of single loads, and the lanes of a wave cover whole cache lines.
__device__ __forceinline__ float2 ld_f2(const float* p) {
    const unsigned long long w = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float2(__int_as_float((int)(unsigned)w), __int_as_float((int)(unsigned)(w >> 32)));
}
__device__ __forceinline__ void ld_f4(const float* p, float* v) {
    const float2 a = ld_f2(p), b = ld_f2(p + 2);
    v[0] = a.x; v[1] = a.y; v[2] = b.x; v[3] = b.y;
}
__device__ __forceinline__ void st_f(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int ld_i(const int* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_i(int* p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// A float that carries the epoch it was written in: one 64-bit store, so a reader that sees the tag sees the value.
__device__ __forceinline__ void st_tagged(unsigned long long* p, float v, unsigned tag) {
    __hip_atomic_store(p, ((unsigned long long)tag << 32) | (unsigned)__float_as_int(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Block k of die `die`'s copy of the exchange arrays (MegaParams::xblk): a few scalar operations when die and k are uniform.
// The kernel keeps the table in scalars of its own, read from the arguments once and made opaque: values the compiler
// knows to be kernel arguments are fetched again from memory wherever registers are short, a scalar load and a wait in
// every phase.
constexpr int kXbQkv = 0, kXbStats = 3, kXbX = 5, kXbX2 = 7, kXbOacc = 9, kXbBar = 10, kXbCount = 11;
__device__ __forceinline__ char* xblock_of(char* base, unsigned long long w0, unsigned long long w1, int k) {
    return base + (size_t)((unsigned)((k < 8 ? w0 : w1) >> (8 * (k & 7))) & 0xFFu) * 8192u;
}
__device__ __forceinline__ unsigned long long ld_u64(const unsigned long long* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Called once per unsuccessful poll (wave-uniform): gives up when the limit is reached (raising the error flag) or when
// another waiter has already raised it, so that one lost workgroup costs one time-out and not one per wait.
__device__ __forceinline__ bool spin_should_stop(int it, int* err) {
    if (it % kMegaErrPeriod != 0) return false;
    if (ld_i(err) == 1) return true;
    if (it >= kMegaSpinLimit) { st_i(err, 1); return true; }
    return false;
}
// Polls two tagged words until both carry `tag` in every active lane of the wave (bounded: raises the error flag).
__device__ __forceinline__ void poll_tagged2(const unsigned long long* a, const unsigned long long* b, unsigned tag,
                                             int* err, float& fa, float& fb) {
    unsigned long long w0 = 0, w1 = 0;
    int it = 0;
    for (;;) {
        w0 = ld_u64(a);
        w1 = ld_u64(b);
        const bool ok = (unsigned)(w0 >> 32) == tag && (unsigned)(w1 >> 32) == tag;
        if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
        if (spin_should_stop(++it, err)) break;
    }
    fa = __int_as_float((int)(unsigned)w0);
    fb = __int_as_float((int)(unsigned)w1);
}

// Polls one tagged word per lane until it carries `tag` in every active lane of the wave (bounded likewise).
__device__ __forceinline__ float poll_tagged1(const unsigned long long* a, unsigned tag, int* err) {
    unsigned long long w0 = 0;
    int it = 0;
    for (;;) {
        w0 = ld_u64(a);
        if (__builtin_amdgcn_ballot_w64((unsigned)(w0 >> 32) != tag) == 0) break;
        if (spin_should_stop(++it, err)) break;
    }
    return __int_as_float((int)(unsigned)w0);
}

typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
// Polls the 2048 tagged words at `base` (the residual stream) with all eight waves until every word carries `tag`, and
// leaves elements 4t..4t+3 in v.  Each load instruction of a wave covers 128 consecutive words, i.e. sixteen whole
// lines: a line is asked for once per round and workgroup (four consecutive words per lane would touch every line with
// four instructions), and what limits this hand-over is the number of poll requests the memory side has to serve.
// A lane's 16-byte load holds two tagged words of one 64-byte sector; each carries its own tag and was written by one
// 8-byte store, so each is seen whole or not at all (the two need not be of the same moment).
// The values then change places inside the wave through its own 1 KiB of LDS (`wave_lds`: 256 floats, no workgroup
// barrier).  A lane that has its values stops loading (its later polls are masked out), so the traffic shrinks as the
// data arrives.  Bounded like every wait here.
__device__ __forceinline__ void poll_tagged4(const unsigned long long* base, unsigned tag, int* err, float* wave_lds, float (&v)[4]) {
    const int lane = threadIdx.x & 63;
    const unsigned long long* p = base + (threadIdx.x >> 6) * 256 + 2 * lane;
    u64x2 w0 = {0, 0}, w1 = {0, 0};
    bool ok = false;
    int it = 0;
    for (;;) {
        if (!ok) {
            // two 16-byte loads per lane, 128 consecutive words per instruction; each 8-byte word inside is read whole
            asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %2, off offset:1024 sc1\n\ts_waitcnt vmcnt(0)"
                         : "=&v"(w0), "=&v"(w1) : "v"(p) : "memory");
            ok = (unsigned)(w0[0] >> 32) == tag && (unsigned)(w0[1] >> 32) == tag && (unsigned)(w1[0] >> 32) == tag &&
                 (unsigned)(w1[1] >> 32) == tag;
        }
        if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
        if (spin_should_stop(++it, err)) break;
    }
    reinterpret_cast<float2*>(wave_lds)[lane] = make_float2(__int_as_float((int)(unsigned)w0[0]), __int_as_float((int)(unsigned)w0[1]));
    reinterpret_cast<float2*>(wave_lds)[64 + lane] = make_float2(__int_as_float((int)(unsigned)w1[0]), __int_as_float((int)(unsigned)w1[1]));
    __builtin_amdgcn_wave_barrier();                 // same wave: its LDS accesses are performed in program order
    const float4 mine = reinterpret_cast<const float4*>(wave_lds)[lane];
    v[0] = mine.x; v[1] = mine.y; v[2] = mine.z; v[3] = mine.w;
}

// Read-only data at a wave-uniform address (layer table, per-row weight scales): the constant address space
// makes these scalar loads, off the vector-memory queue.
__device__ __forceinline__ float ldc_f(const float* p) { return *(const float __attribute__((address_space(4)))*)(uintptr_t)p; }

__device__ __forceinline__ LayerW4 ldc_layer4(const LayerW4* p) {
    static_assert(sizeof(LayerW4) == 12 * sizeof(unsigned long long), "LayerW4 is twelve pointers");
    const unsigned long long __attribute__((address_space(4)))* q = (const unsigned long long __attribute__((address_space(4)))*)(uintptr_t)p;
    LayerW4 w;
    w.wqkv = (int8_t*)q[0]; w.wo = (int8_t*)q[1]; w.wgu = (int8_t*)q[2]; w.wd = (int8_t*)q[3];
    w.sqkv = (float*)q[4]; w.so = (float*)q[5]; w.sgu = (float*)q[6]; w.sd = (float*)q[7];
    w.mqkv = (float*)q[8]; w.mo = (float*)q[9]; w.mgu = (float*)q[10]; w.md = (float*)q[11];
    return w;
}
__device__ __forceinline__ LayerW ldc_layer(const LayerW* p) {
    static_assert(sizeof(LayerW) == 8 * sizeof(unsigned long long), "LayerW is eight pointers");
    const unsigned long long __attribute__((address_space(4)))* q = (const unsigned long long __attribute__((address_space(4)))*)(uintptr_t)p;
    LayerW w;
    w.wqkv = (int8_t*)q[0]; w.wo = (int8_t*)q[1]; w.wgu = (int8_t*)q[2]; w.wd = (int8_t*)q[3];
    w.sqkv = (float*)q[4]; w.so = (float*)q[5]; w.sgu = (float*)q[6]; w.sd = (float*)q[7];
    return w;
}

// Grid barrier from device-scope relaxed atomics: workgroup w adds 1 to the counter of group w mod 8 (8 counters on
// separate 256-byte lines, so at most 32 atomics serialise on one address) and the last arriver of a group publishes
// the epoch in the group's release flag; wave 0 of every workgroup polls the eight flags, one lane each.  Every flag
// exists in eight copies and workgroup w polls copy w mod 8 of each: a store into a line that 256 workgroups are
// polling queues behind their loads at the memory side, behind 32 pollers it lands sooner.  One atomic round trip and
// one store-to-poll hand-over from the last arrival to the release (a top-level counter between the groups and one
// flag adds a second round trip: +4 us per token; 16 groups of 16 or 4 of 64: +2).  (Polling the group counters
// directly costs more: 256 pollers then contend with the arriving atomics on the same lines.  A barrier without
// atomics - every workgroup stores the epoch into a word of its own in each of the eight copies and polls all 256
// words of its copy - costs more as well: +1 us per layer.)
// Workgroups are dealt to the XCDs round-robin, so group g and the pollers of copy g are the 32 workgroups of XCD g:
// its counter and its flag copies live in memory of that XCD's die (mem[die]).  Which block a word is in follows from
// the static index and die_mask alone, never from where a workgroup really runs: writers and pollers always agree.
struct GridBarrier {
    unsigned* mem[2];                           // per die: [64 g] group counters, [kMegaFlagBase + 16 (8 r + g)] copy r of group g's release flag
    unsigned die_mask;
    unsigned epoch;
    int* err;
    bool dead = false;                          // wave 0 only: a wait timed out or the error flag was seen; later waits return at once
    __device__ __forceinline__ unsigned* block_of(int xcd) const { return ((die_mask >> xcd) & 1u) ? mem[1] : mem[0]; }
    // drain == false: the calling wave made no global store in this phase and may keep loads in flight
    __device__ __forceinline__ void arrive(bool drain = true) {
        if (drain) __builtin_amdgcn_s_waitcnt(0);          // this thread's stores have been acknowledged
        __syncthreads();
        epoch++;
        if (threadIdx.x < 64) {
            bool last = false;
            const int g = blockIdx.x % kMegaGroups;
            if (threadIdx.x == 0) {
                const unsigned old = __hip_atomic_fetch_add(&block_of(g)[64 * g], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                last = old == epoch * kMegaGroup - 1;
            }
            if (__builtin_amdgcn_ballot_w64(last) != 0) {        // the group is complete: its flag, in all copies
                const int r = threadIdx.x;
                if (r < kMegaFlagCopies)
                    __hip_atomic_store(&block_of(r)[kMegaFlagBase + 16 * (kMegaGroups * r + g)], epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    __device__ __forceinline__ void wait() {
        if (threadIdx.x < 64 && !dead) {
            // lane j polls group j's flag, in this workgroup's copy
            const int r = blockIdx.x % kMegaFlagCopies;
            const unsigned* flag = &block_of(r)[kMegaFlagBase + 16 * (kMegaGroups * r + threadIdx.x % kMegaGroups)];
            int it = 0;
            for (;;) {
                // signed distance so that the comparison survives counter wrap-around
                const bool behind = (int)(__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - epoch) < 0;
                if (__builtin_amdgcn_ballot_w64(behind) == 0) break;
                if (spin_should_stop(++it, err)) { dead = true; break; }
            }
        }
        __syncthreads();
    }
};

struct MegaLds {
    __attribute__((aligned(16))) float f[8192];        // FHT buffer / fp32 staging (32 KiB)
    __attribute__((aligned(16))) int8_t xq[8192];      // quantised activation vector of the current GEMV
    float red[kMegaWaves];                             // two-barrier reductions of the lm_head section
    float red_min[kMegaWaves];                         // W4A4: the minimum of the asymmetric quantiser
    float red_sum[kMegaWaves], red_max[kMegaWaves];    // one-barrier reductions (a slot is rewritten only several barriers after its last read)
    float sc[4][kChunk];                               // scores of this chunk, 4 query heads
    __attribute__((aligned(16))) int8_t q8[4][kHd];
    __attribute__((aligned(16))) int8_t knew[kHd];
    __attribute__((aligned(16))) int8_t vnew[kHd];
    __attribute__((aligned(16))) uint8_t pb[4][kChunk];
    float rowmax[4], rowcd[4];
    int osum[4][kHd];
    float bestv[kMegaWaves];
    int besti[kMegaWaves];
    float hst[32];                                     // SiLU(gate)*up of this workgroup's 32 row pairs, stream waves -> store wave
    float res8[8];                                     // the workgroup's eight o_proj / down outputs, gathered for one store
    float tk_val[kTopKMax];                            // sampling: the selected candidates (this workgroup's, then the global ones)
    int tk_idx[kTopKMax];
    int tk_tok;
    int stop;                                          // set by thread 0 at the end of a step when the error flag is up: the launch ends there
#ifdef FX_MEGA_ALL_STAMPS
    long long dbg[12];                                 // debug build: the stamps of one layer, stored to memory at the layer's end
#endif
    __attribute__((aligned(16))) int8_t wd[8][8192];   // this workgroup's 8 down rows, filled by global->LDS direct loads (64 KiB);
                                                       // the odd rows first hold gate/up rows 12..15 of their stream wave
    __attribute__((aligned(16))) int8_t gu2[4][8192];  // gate/up rows 8..11 of each stream wave (32 KiB)
};

template <int NW>
__device__ __forceinline__ float mega_block_max(float v, float* red) { return block_max<NW>(v, red); }

template <class Hook>
__device__ __forceinline__ float mega_block_sum(float v, float* slot, Hook hook) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    __syncthreads();
    hook();
    float r = slot[0];
#pragma unroll
    for (int i = 1; i < kMegaWaves; i++) r += slot[i];
    return r;
}
template <class Hook>
__device__ __forceinline__ float mega_block_max_h(float v, float* slot, Hook hook) {
    v = wave_max(v);
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    __syncthreads();
    hook();
    float r = slot[0];
#pragma unroll
    for (int i = 1; i < kMegaWaves; i++) r = fmaxf(r, slot[i]);
    return r;
}
struct NoHook { __device__ __forceinline__ void operator()() const {} };

// RMSNorm (optional) + per-token int8 quantisation of a 2048-vector held as 4 values per thread; result in L.xq.
// Returns the quantisation scale to every thread.
// `hook` runs in every thread right after the first workgroup barrier, i.e. once every wave's activation loads
// have been consumed: the stream waves issue their next slice of weight prefetch there.
template <class Hook>
__device__ __forceinline__ float norm_quant_2048(float (&v)[4], const float4& g, bool do_norm, float eps,
                                                 MegaLds& L, Hook hook) {
    const int t = threadIdx.x;
    if (do_norm) {
        float ss = (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
        ss = mega_block_sum(ss, L.red_sum, hook);
        const float rms = 1.0f / sqrtf(ss / 2048.0f + eps);
        v[0] = v[0] * rms * g.x; v[1] = v[1] * rms * g.y; v[2] = v[2] * rms * g.z; v[3] = v[3] * rms * g.w;
    }
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    if (do_norm) amax = mega_block_max_h(amax, L.red_max, NoHook());
    else amax = mega_block_max_h(amax, L.red_max, hook);
    const float sc = sym_scale_127_uniform(amax);
    int n[4];
    quant_vector(v, sc, n);
    reinterpret_cast<uint32_t*>(L.xq)[t] = pack4_i8(n[0], n[1], n[2], n[3]);
    __syncthreads();
    return sc;
}

template <class Hook>
__device__ __forceinline__ float mega_block_min_h(float v, float* slot, Hook hook) {
    v = wave_min(v);
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
    __syncthreads();
    hook();
    float r = slot[0];
#pragma unroll
    for (int i = 1; i < kMegaWaves; i++) r = fminf(r, slot[i]);
    return r;
}
// N values of a thread (N = 4: consecutive elements 4t..; N = 16: four groups of four consecutive ones) quantised to
// asymmetric uint4 with the given minimum and scale, the arithmetic of quant_asym_kernel: round((x - min) / s) & 15,
// packed low nibble first.  Returns one 16-bit word per group of four.
template <int N>
__device__ __forceinline__ void quant_u4_pack(const float (&v)[N], float vmin, float sc, uint16_t (&out)[N / 4]) {
    float d[N];
    int n[N];
#pragma unroll
    for (int i = 0; i < N; i++) d[i] = v[i] - vmin;
    quant_vector(d, sc, n);
#pragma unroll
    for (int g = 0; g < N / 4; g++)
        out[g] = (uint16_t)((n[4 * g] & 15) | ((n[4 * g + 1] & 15) << 4) | ((n[4 * g + 2] & 15) << 8) | ((n[4 * g + 3] & 15) << 12));
}
// W4A4 counterpart of norm_quant_2048: RMSNorm (optional) + per-token asymmetric uint4 quantisation; the packed vector
// (1024 bytes) goes to L.xq, the scale comes back in .x and the zero point (the minimum) in .y.
template <class Hook>
__device__ __forceinline__ float2 norm_quant_2048_u4(float (&v)[4], const float4& g, bool do_norm, float eps,
                                                     MegaLds& L, Hook hook) {
    const int t = threadIdx.x;
    if (do_norm) {
        float ss = (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
        ss = mega_block_sum(ss, L.red_sum, hook);
        const float rms = 1.0f / sqrtf(ss / 2048.0f + eps);
        v[0] = v[0] * rms * g.x; v[1] = v[1] * rms * g.y; v[2] = v[2] * rms * g.z; v[3] = v[3] * rms * g.w;
    }
    float vmax = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
    float vmin = fminf(fminf(v[0], v[1]), fminf(v[2], v[3]));
    if (do_norm) vmax = mega_block_max_h(vmax, L.red_max, NoHook());
    else vmax = mega_block_max_h(vmax, L.red_max, hook);
    vmin = mega_block_min_h(vmin, L.red_min, NoHook());
    float sc = (vmax - vmin) / 15.0f;
    if (sc == 0.0f) sc = 1.0f;
    uint16_t w16[1];
    quant_u4_pack(v, vmin, sc, w16);
    reinterpret_cast<uint16_t*>(L.xq)[t] = w16[0];
    __syncthreads();
    return make_float2(sc, vmin);
}
// One packed row against the packed activation vector in LDS: the unsigned activations enter the signed 4-bit dot
// product as a - 8, and 8 x (row sum of the weights, a second dot product with ones) is added back.
template <int NCH>
__device__ __forceinline__ int mega_dot_row4(const i32x4 (&wr)[NCH], const int8_t* xq_lds, int lane) {
    const i32x4 ones = {0x11111111, 0x11111111, 0x11111111, 0x11111111};
    int acc = 0, wsum = 0;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        i32x4 xs = reinterpret_cast<const i32x4*>(xq_lds)[lane + 64 * i];
        xs.x ^= 0x88888888; xs.y ^= 0x88888888; xs.z ^= 0x88888888; xs.w ^= 0x88888888;
        acc = dot32_i4(wr[i], xs, acc);
        wsum = dot32_i4(wr[i], ones, wsum);
    }
    return wave_sum_i(acc + 8 * wsum);
}
// One 4096-byte packed weight row (K = 8192) from global memory straight into LDS, as mega_row_to_lds.
__device__ __forceinline__ void mega_row4_to_lds(const int8_t* __restrict__ w, int row, int lane, int8_t* lds_row) {
    const int8_t* base = w + (size_t)row * 4096;
    const unsigned voff = lane * 16;
    const unsigned dst = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)lds_row);
    unsigned saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\t"
                 "s_mov_b32 m0, %3\n\t"
                 "s_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %2\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:1024\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:2048\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:3072\n\t"
                 "s_mov_b32 m0, %0"
                 : "=&s"(saved_m0) : "v"(voff), "s"(base), "s"(dst) : "memory");
}
__device__ __forceinline__ int mega_dot_row4_lds(const int8_t* w_lds, const int8_t* xq_lds, int lane) {
    i32x4 wr[4];
#pragma unroll
    for (int i = 0; i < 4; i++) wr[i] = reinterpret_cast<const i32x4*>(w_lds)[lane + 64 * i];
    return mega_dot_row4<4>(wr, xq_lds, lane);
}

// Weight rows are read through a pointer that is explicitly in the global address space: a generic pointer
// would make these FLAT loads, which also count on the LDS/scalar counter, and every LDS wait of the wave
// would then wait for the weight prefetch as well.
typedef const i32x4 __attribute__((address_space(1)))* global_i32x4_ptr;
template <int NCH>
__device__ __forceinline__ void mega_load_rows(const int8_t* __restrict__ w, int k, int row, int lane, i32x4 (&wr)[NCH]) {
    const global_i32x4_ptr p = (global_i32x4_ptr)(uintptr_t)(w + (size_t)row * k);
#pragma unroll
    for (int i = 0; i < NCH; i++) wr[i] = __builtin_nontemporal_load(p + lane + 64 * i);
}
// One 8192-byte weight row straight from global memory into LDS (16 bytes per lane, lane i of chunk c lands
// at byte 1024*c + 16*i): no registers are held while the row is in flight.  Counts on the vector-memory
// counter like a load; the issuing wave waits for that counter to reach zero before it reads the row.
// Issued from inline assembly on purpose: for the builtin form the compiler makes every later LDS access that
// it cannot prove disjoint (all of them here) wait for the transfer, which stalls the issuing wave at once.
// Loads the compiler does not know of only make its own counter waits stricter, never too lax: results
// return in issue order.
__device__ __forceinline__ void mega_row_to_lds(const int8_t* __restrict__ w, int row, int lane, int8_t* lds_row) {
    // scalar base + one 32-bit lane offset; the instruction offset advances the global and the LDS address alike
    const int8_t* base = w + (size_t)row * 8192;
    const unsigned voff = lane * 16;
    const unsigned dst = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)lds_row);
    unsigned saved_m0;
#pragma unroll
    for (int half = 0; half < 2; half++)
        asm volatile("s_mov_b32 %0, m0\n\t"
                     "s_mov_b32 m0, %3\n\t"
                     "s_nop 0\n\t"
                     "global_load_lds_dwordx4 %1, %2\n\t"
                     "global_load_lds_dwordx4 %1, %2 offset:1024\n\t"
                     "global_load_lds_dwordx4 %1, %2 offset:2048\n\t"
                     "global_load_lds_dwordx4 %1, %2 offset:3072\n\t"
                     "s_mov_b32 m0, %0"
                     : "=&s"(saved_m0) : "v"(voff), "s"(base + 4096 * half), "s"(dst + 4096u * half) : "memory");
}
__device__ __forceinline__ int mega_dot_row_lds(const int8_t* w_lds, const int8_t* xq_lds, int lane) {
    int acc = 0;
#pragma unroll
    for (int i = 0; i < 8; i++)
        acc = dot16(reinterpret_cast<const i32x4*>(w_lds)[lane + 64 * i], reinterpret_cast<const i32x4*>(xq_lds)[lane + 64 * i], acc);
    return wave_sum_i(acc);
}

template <int NCH>
__device__ __forceinline__ int mega_dot_row(const i32x4 (&wr)[NCH], const int8_t* xq_lds, int lane) {
    int acc = 0;
#pragma unroll
    for (int i = 0; i < NCH; i++) acc = dot16(wr[i], reinterpret_cast<const i32x4*>(xq_lds)[lane + 64 * i], acc);
    return wave_sum_i(acc);
}

// W4 = false: W8A8 (symmetric int8 activations and weights).  W4 = true: the W4A4 configuration (asymmetric uint4
// activations, int4 weights two per byte, int4 output head); attention, exchanges and wave roles are the same, the
// weight rows are half as long: a stream wave then holds all 16 of its gate/up rows in registers.
template <bool W4>
__device__ __forceinline__ void decode_mega_body(const MegaParams& p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char mega_smem[];   // sizeof(MegaLds) > the static 64 KiB limit
    MegaLds& L = *reinterpret_cast<MegaLds*>(mega_smem);
    const int t = threadIdx.x, wg = blockIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const bool is_s = wave >= 4;                        // stream wave (see the file comment)
    const int sw = wave - 4;
    constexpr int H = 2048, KV = 512, QH = 32, KVH = 8, GROUP = 4;
    char* xbase = p.xarena;
    unsigned long long xw00 = p.xblk[0][0], xw01 = p.xblk[0][1], xw10 = p.xblk[1][0], xw11 = p.xblk[1][1];
    asm volatile("" : "+s"(xbase), "+s"(xw00), "+s"(xw01), "+s"(xw10), "+s"(xw11));
    struct XT {} xt;                                             // (tag for the two accessors below)
    auto xblock = [&](XT, int die_, int k) -> char* { return xblock_of(xbase, die_ ? xw10 : xw00, die_ ? xw11 : xw01, k); };
    auto xwords = [&](XT, int die_, int k) -> unsigned long long* { return reinterpret_cast<unsigned long long*>(xblock(xt, die_, k)); };
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // see MegaParams::h
    // The launch state was left by the previous launch (or a small kernel before this one).  It is read with coherent
    // loads: the compiler would otherwise fetch it through the scalar cache, whose requests do not queue behind the
    // invalidation above and could be served from a line of an earlier launch that survived in this XCD's L2.
    const int pos0 = ld_i(&p.state[0]);
    const int step_base = ld_i(&p.state[1]);
    GridBarrier bar{{reinterpret_cast<unsigned*>(xblock(xt, 0, kXbBar)), reinterpret_cast<unsigned*>(xblock(xt, 1, kXbBar))}, p.die_mask,
                    (unsigned)ld_i(&p.state[2]), &p.state[3]};
    const unsigned seq0 = (unsigned)ld_i(&p.state[4]);
    int stamp_i = 0;
    // 'thread 0 of workgroup 0' from scalars and the hardware lane id: no per-thread value has to stay live for it
    auto is_t0 = [&]() { return wave == 0 && __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)) == 0; };
#ifdef FX_MEGA_ALL_STAMPS
    // debug build: every workgroup records the 12 stamps of one layer (the eighth) behind the other timeline entries.
    // They wait in LDS until the layer's last one: a store per stamp would sit in front of the next wait for the
    // vector-memory counter and stretch exactly the intervals under study (by up to 1 us).  No other stamps in this build.
    int cur_layer = 0;
    auto stamp = [&]() {
        if (p.timeline && is_t0() && cur_layer == 8) {
            L.dbg[stamp_i % 12] = wall_clock64();
            if (stamp_i % 12 == 11)
                for (int i = 0; i < 12; i++) p.timeline[p.n_layers * 12 + 2 + 64 + 2 * kMegaWG + wg * 12 + i] = L.dbg[i];
        }
        stamp_i++;
    };
#else
    auto stamp = [&]() { if (p.timeline && wg == p.timeline_wg && is_t0()) p.timeline[stamp_i] = wall_clock64(); stamp_i++; };
#endif
#ifdef FX_MEGA_FINE_STAMPS
    int fine_i = 0;
    auto fine = [&]() { if (p.timeline && wg == 0 && is_t0() && fine_i < 64) p.timeline[p.n_layers * 12 + 2 + fine_i] = wall_clock64(); fine_i++; };
    if (p.timeline && is_t0()) p.timeline[p.n_layers * 12 + 2 + 64 + wg] = wall_clock64();               // workgroup entry
#else
    auto fine = [&]() {};
#endif
    int tok = p.x_in ? 0 : ld_i(&p.token[0]);
    if ((unsigned)tok >= (unsigned)p.vocab) {                      // never look up a row outside the table: report and use token 0
        if (wg == 0 && threadIdx.x == 0) st_i(&p.state[3], 2);
        tok = 0;
    }
    const bool greedy = p.tokens_out != nullptr;
    const bool sampling = greedy && p.top_k > 0;

    // Greedy mode runs several tokens in one launch: after the lm_head every workgroup reduces the per-workgroup
    // candidates itself, so all of them know the next token and position without a further exchange.
    int steps_done = 0, stop = 0;
    for (int step = 0; step < p.n_steps && !stop; step++) {
    const int pos = pos0 + step;
    const int len = pos + 1;
    stamp_i = 0;                                                  // a timeline holds the stamps of the last step

    // attention work item of this workgroup
    const int a_h = wg / 32, a_c = wg % 32;
    // The die this workgroup really runs on: it only chooses which copy to READ, and both copies hold the same words.
    int die;
    {
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        die = (int)((p.die_mask >> (xcc & 7u)) & 1u);
    }
    // this wave's 256 words of its die's copy, as poll_tagged4 addresses them (base + wave * 256)
    auto my_copy = [&](int xb) -> const unsigned long long* { return xwords(xt, die, xb + (wave >> 2)) - (wave >> 2) * 1024; };
    // the eight values of this workgroup go to both copies: threads 0..7 write copy 0, threads 8..15 copy 1
    auto publish8 = [&](int xb, const float* v8, unsigned tag_) {
        const int t_ = threadIdx.x;
        if (t_ < 16) st_tagged(xwords(xt, t_ >> 3, xb + (wg >> 7)) + (wg & 127) * 8 + (t_ & 7), v8[t_ & 7], tag_);
    };
    const bool a_active = a_c * kChunk < len && a_c * kChunk < p.max_pos;
    const bool a_owner = a_active && (pos / kChunk == a_c);       // this chunk holds the new token
    const int nchunks = (len + kChunk - 1) / kChunk;              // active chunks per head: the parts every accumulator receives

    for (int l = 0; l < p.n_layers; l++) {
        // An opaque per-layer copy of the thread index: without it the compiler hoists every per-thread address
        // offset of all phases out of the layer loop, and the ~100 registers they occupy push the prefetched
        // weights into scratch memory.
        int t_opaque = threadIdx.x;
        asm volatile("" : "+v"(t_opaque));
        const int t = t_opaque, lane = t & 63;
#ifdef FX_MEGA_ALL_STAMPS
        cur_layer = l;
#endif
        typename std::conditional<W4, LayerW4, LayerW>::type w;
        if constexpr (W4) w = ldc_layer4(reinterpret_cast<const LayerW4*>(p.layers) + l);
        else w = ldc_layer(reinterpret_cast<const LayerW*>(p.layers) + l);
        // sequence number of this layer pass: unique over launches, the tag of everything this pass publishes
        const unsigned tag = seq0 + (unsigned)(step * p.n_layers + l) + 1u;
        const float* g0 = p.gamma + (size_t)(2 * l) * H;
        const float* g1 = p.gamma + (size_t)(2 * l + 1) * H;
        const float* q_s = p.q_s + l * QH;
        const float* k_s = p.k_s + l * KVH;
        const float* v_s = p.v_s + l * KVH;
        const float* a_s = p.a_s + l * QH;
        int8_t* kc = p.k_cache + (size_t)l * p.cache_layer_bytes;
        int8_t* vc = p.v_cache + (size_t)l * p.cache_layer_bytes;
        // h of this layer pass lives at an address that no other pass of this launch uses (see MegaParams::h)
        float* hbuf = p.h + (size_t)(step * p.n_layers + l) * 8192;

        // Stream waves: 16 gate/up rows (interleaved gate, up) and 2 down rows each, fetched in six slices of
        // 8 KiB per wave, one per phase, each issued once the phase's activation loads have landed.  A slice
        // (8 MiB over the chip) drains while the phase computes; issuing a whole matrix at once instead fills
        // the memory queues for microseconds, and the barrier's own round trips then queue behind it.
        // Slices 0 and 1 (rows 0..7) wait in registers, slices 2 and 3 and the down rows in LDS.
        // (W4A4: 16 rows of 1024 bytes each, all of them in registers, four per slice: gu[r >> 1][r & 1] is row r.)
        i32x4 gu[8][2];
        // Only the stream waves ever define these registers.  An empty asm "defines" them for every wave here,
        // or the compiler would carry the stale values of the other waves around the layer and token loops.
#pragma unroll
        for (int r = 0; r < 8; r++) asm volatile("" : "=v"(gu[r][0]), "=v"(gu[r][1]));
        auto gu_slice = [&](int s) {
            if constexpr (W4) {
                __builtin_amdgcn_s_waitcnt(0x0F70);            // vmcnt(0) only, as below
                if (is_s) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        i32x4 one[1];
                        mega_load_rows<1>(w.wgu, H / 2, wg * 64 + sw * 16 + 4 * s + r, lane, one);
                        gu[(4 * s + r) >> 1][(4 * s + r) & 1] = one[0];
                    }
                }
                return;
            }
            // Every wave first waits for its own older loads (long landed at the points where this is called).
            // Otherwise the wait inserted for such a load after the branch below has to assume the path without
            // the slice, and it would make the stream waves sit out their own prefetch.
            __builtin_amdgcn_s_waitcnt(0x0F70);            // vmcnt(0) only
            if (is_s) {
                if (s < 2) {
#pragma unroll
                    for (int r = 0; r < 4; r++) mega_load_rows<2>(w.wgu, H, wg * 64 + sw * 16 + 4 * s + r, lane, gu[(4 * s + r) & 7]);
                } else {
                    // four consecutive 2048-byte rows are one 8192-byte run
                    mega_row_to_lds(w.wgu, wg * 16 + sw * 4 + s, lane, s == 2 ? L.gu2[sw] : L.wd[sw * 2 + 1]);
                }
            }
        };

        // ================= phase 1: RMSNorm + quant -> q/k/v rows (12 per workgroup, 3 per wave 0..3) =================
        {
            i32x4 wr[3][2];
            float wsc[3] = {0.0f, 0.0f, 0.0f}, wsm[3] = {0.0f, 0.0f, 0.0f};
            if (!is_s) {
#pragma unroll
                for (int j = 0; j < 3; j++) {
                    if constexpr (W4) {
                        i32x4 one[1];
                        mega_load_rows<1>(w.wqkv, H / 2, wg * 12 + wave + 4 * j, lane, one);
                        wr[j][0] = one[0];
                        wsm[j] = ldc_f(w.mqkv + wg * 12 + wave + 4 * j);
                    } else {
                        mega_load_rows<2>(w.wqkv, H, wg * 12 + wave + 4 * j, lane, wr[j]);
                    }
                    wsc[j] = ldc_f(w.sqkv + wg * 12 + wave + 4 * j);
                }
            }
            const float4 gam = reinterpret_cast<const float4*>(g0)[t];
            float v[4];
            if (l > 0) poll_tagged4(my_copy(kXbX), tag - 1u, bar.err, L.f + (t >> 6) * 256, v);   // x of the previous layer, as it arrives
            stamp();
            if (l == 0) {
                if (p.x_in) { const float4 q = reinterpret_cast<const float4*>(p.x_in)[t]; v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w; }
                else {
#pragma unroll
                    for (int i = 0; i < 4; i++) v[i] = __half2float(p.embed[(size_t)tok * H + 4 * t + i]);
                }
            }
            float sx, bx = 0.0f;
            if constexpr (W4) { const float2 sb = norm_quant_2048_u4(v, gam, true, p.eps, L, [&]() { gu_slice(0); }); sx = sb.x; bx = sb.y; }
            else sx = norm_quant_2048(v, gam, true, p.eps, L, [&]() { gu_slice(0); });
            if (!is_s) {
#pragma unroll
                for (int j = 0; j < 3; j++) {
                    const int r = wg * 12 + wave + 4 * j;
                    float out;
                    if constexpr (W4) {
                        const i32x4 one[1] = {wr[j][0]};
                        out = (float)mega_dot_row4<1>(one, L.xq, lane) * sx * wsc[j];
                        out = out + bx * wsm[j];
                    } else {
                        out = (float)mega_dot_row<2>(wr[j], L.xq, lane) * sx * wsc[j];
                    }
                    if (lane < 2) st_tagged(xwords(xt, lane, kXbQkv + (r >> 10)) + (r & 1023), out, tag);   // lane 0 -> copy 0, lane 1 -> copy 1
                }
            }
            stamp();
            // no grid barrier here: a KV head's 32 workgroups need 384 of the 3072 outputs and poll their tagged words
        }

        // ================= phase 2: RoPE/quant/append, scores of this chunk, chunk statistics =================
        {
            // (Requesting these cache rows any earlier does not pay: ahead of the poll for x they hold that poll's
            // answers up, which return in issue order, and from phase 6 of the layer before they slow that phase.)
            i32x4 kreg = {0, 0, 0, 0};
            const int key = t >> 2, part = t & 3;
            const int kpos = a_c * kChunk + key;
            if (a_active) kreg = *reinterpret_cast<const i32x4*>(kc + k_index(a_h, min(kpos, p.max_pos - 1), p.max_pos) + part * 16);
            // this chunk's V block for the second half of the phase (d = channel, 16 positions per thread)
            i32x4 vreg = {0, 0, 0, 0};
            const int blk = t >> 8, d = (t >> 2) & 63;
            const int bpos = a_c * kChunk + blk * kVBlock;
            if (a_active && bpos < p.max_pos)
                vreg = *reinterpret_cast<const i32x4*>(vc + v_index(a_h, bpos, d, p.max_pos) + part * 16);
            const float as_g = ldc_f(a_s + a_h * GROUP + (wave >> 1));   // threads 128g..128g+127 (two waves) serve query head g
            // static scales of this layer, read ahead of the barrier (and of this phase's prefetch slice)
            float qs4[GROUP];
#pragma unroll
            for (int g = 0; g < GROUP; g++) qs4[g] = ldc_f(q_s + a_h * GROUP + g);
            const float ks1 = ldc_f(k_s + a_h), vs1 = ldc_f(v_s + a_h);
            if (a_active) {
                const float* sn = p.rope_sin + (size_t)pos * 32;
                const float* cs = p.rope_cos + (size_t)pos * 32;
                if (t < 128) {                                        // q: 4 heads x 32 pairs
                    const int g = t >> 5, k = t & 31, qh = a_h * GROUP + g;
                    float t0, t1;
                    const unsigned long long* src = xwords(xt, die, kXbQkv + (a_h >> 2)) + (qh * kHd & 1023) + k;   // 16 heads per block
                    poll_tagged2(src, src + 32, tag, bar.err, t0, t1);
                    const float o0 = t0 * cs[k] - t1 * sn[k], o1 = t0 * sn[k] + t1 * cs[k];
                    const float div = 8.0f * (g == 0 ? qs4[0] : g == 1 ? qs4[1] : g == 2 ? qs4[2] : qs4[3]);
                    L.q8[g][k] = (int8_t)static_q8(o0, div);
                    L.q8[g][k + 32] = (int8_t)static_q8(o1, div);
                } else if (t < 160) {                                 // k of the new token: 32 pairs
                    const int k = t - 128;
                    float t0, t1;
                    const unsigned long long* src = xwords(xt, die, kXbQkv + 2) + a_h * kHd + k;       // block 2: k, then v
                    poll_tagged2(src, src + 32, tag, bar.err, t0, t1);
                    const float o0 = t0 * cs[k] - t1 * sn[k], o1 = t0 * sn[k] + t1 * cs[k];
                    const float div = 1.0f * ks1;
                    const int8_t b0 = (int8_t)static_q8(o0, div), b1 = (int8_t)static_q8(o1, div);
                    L.knew[k] = b0; L.knew[k + 32] = b1;
                    if (a_owner) { int8_t* dst = kc + k_index(a_h, pos, p.max_pos); dst[k] = b0; dst[k + 32] = b1; }
                } else if (t >= 192 && t < 256) {                     // v of the new token: a wave of its own (two polls in
                    const int d = t - 192;                            // one wave would run one after the other)
                    const float tv = poll_tagged1(xwords(xt, die, kXbQkv + 2) + KV + a_h * kHd + d, tag, bar.err);
                    const int8_t b = (int8_t)static_q8(tv, 1.0f * vs1);
                    L.vnew[d] = b;
                    if (a_owner) vc[v_index(a_h, pos, d, p.max_pos)] = b;
                }
                stamp();
                __syncthreads();
                gu_slice(1);                                          // the q/k/v loads of this phase have landed
                if (kpos == pos) kreg = reinterpret_cast<const i32x4*>(L.knew)[part];
                float s_mine = 0.0f;
#pragma unroll
                for (int g = 0; g < GROUP; g++) {
                    int acc = dot16(kreg, reinterpret_cast<const i32x4*>(L.q8[g])[part], 0);
                    acc += lane_xor_i<1>(acc);
                    acc += lane_xor_i<2>(acc);
                    const float s = (float)acc * qs4[g] * ks1;
                    if (part == g) s_mine = s;
                }
                L.sc[part][key] = kpos < len ? s_mine : -1e32f;
                __syncthreads();
                if (wave < GROUP) {
                    const float s0 = L.sc[wave][lane], s1 = L.sc[wave][lane + 64];
                    const float m = wave_max(fmaxf(s0, s1));
                    float sum = (a_c * kChunk + lane < len ? exp_f(s0 - m) : 0.0f) + (a_c * kChunk + lane + 64 < len ? exp_f(s1 - m) : 0.0f);
                    sum = wave_sum(sum);
                    if (lane < 2) {                                   // lane 0 -> copy 0, lane 1 -> copy 1
                        unsigned long long* slot = xwords(xt, lane, kXbStats + (a_h >> 2)) + (size_t)((a_h & 3) * GROUP + wave) * 64 + a_c;
                        st_tagged(slot, m, tag);
                        st_tagged(slot + 32, sum, tag);
                    }
                }
            } else {
                // A workgroup without a key chunk keeps the pace of the others: its two slices issued at once, right
                // behind phase 1, crowd the q/k/v and statistics hand-overs of the workgroups that have one (-10 us per
                // token at half the maximum context).  The others need longer the more chunks exchange statistics.
                __builtin_amdgcn_s_sleep(40);
                gu_slice(1);
            }
            stamp();
            // ---- second half: row statistics, uint8 probabilities, partial P.V ----
            // The only thing that crosses workgroups between the halves is the pair (max, sum) of every chunk of the
            // same head.  Each value carries the barrier epoch of this phase in its high word, so the 32 workgroups of
            // a KV head poll those words directly instead of going through a grid barrier and a load after it; the
            // slot is next written a layer later, three grid barriers after every reader has finished with it.
            if (a_active) {
                if (wave < GROUP) {
                    float m_c = -1e32f, l_c = 0.0f;
                    {
                        // the maxima of a head's 32 chunks are consecutive words, then its sums: a poll is two loads of whole lines
                        const unsigned long long* slot = xwords(xt, die, kXbStats + (a_h >> 2)) + (size_t)((a_h & 3) * GROUP + wave) * 64 + min(lane, nchunks - 1);
                        unsigned long long w0 = 0, w1 = 0;
                        int it = 0;
                        for (;;) {
                            w0 = ld_u64(slot);
                            w1 = ld_u64(slot + 32);
                            const bool ok = (unsigned)(w0 >> 32) == tag && (unsigned)(w1 >> 32) == tag;
                            if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
                            if (spin_should_stop(++it, bar.err)) break;
                        }
                        if (lane < nchunks) { m_c = __int_as_float((int)(unsigned)w0); l_c = __int_as_float((int)(unsigned)w1); }
                    }
                    const float mx = wave_max(m_c);
                    const float sum = wave_sum(lane < nchunks ? l_c * exp_f(m_c - mx) : 0.0f);
                    if (lane == 0) { L.rowmax[wave] = mx; L.rowcd[wave] = 1.0f / sum; }
                }
                stamp();                                              // workgroup 0 is always active: its timeline keeps 12 stamps per layer
                __syncthreads();
                gu_slice(2);                                          // the chunk statistics have landed
                {
                    const int g = t >> 7, key = t & 127;
                    const float pr = exp_f(L.sc[g][key] - L.rowmax[g]) * L.rowcd[g];
                    int p8 = (int)roundf(pr / (1.0f * as_g));
                    p8 = p8 > 255 ? 255 : p8;
                    if (a_c * kChunk + key >= len) p8 = 0;
                    L.pb[g][key] = (uint8_t)(p8 ^ 0x80);
                }
                // the new token's V row is not in the cache yet: patch it into the prefetched registers
                if (pos >= bpos + part * 16 && pos < bpos + part * 16 + 16) {
                    const int byte = pos & 15;
                    int wsel = vreg[byte >> 2];
                    const int sh = (byte & 3) * 8;
                    wsel = (wsel & ~(0xff << sh)) | (((int)(uint8_t)L.vnew[d]) << sh);
                    vreg[byte >> 2] = wsel;
                }
                __syncthreads();
                const i32x4 ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
                int vsum = dot16(ones, vreg, 0);
                int tot[GROUP];
#pragma unroll
                for (int g = 0; g < GROUP; g++) {
                    int acc = dot16(reinterpret_cast<const i32x4*>(L.pb[g])[blk * 4 + part], vreg, 0) + 128 * vsum;
                    acc += lane_xor_i<1>(acc);
                    acc += lane_xor_i<2>(acc);
                    tot[g] = acc;
                }
                if (blk == 1 && part == 0) {
#pragma unroll
                    for (int g = 0; g < GROUP; g++) L.osum[g][d] = tot[g];
                }
                __syncthreads();
                if (blk == 0 && part == 0) {
#pragma unroll
                    for (int i = 0; i < GROUP; i++) {
                        // the 32 chunks of a KV head add into the same 256 words: each starts at another query head,
                        // so that they do not all queue on the same 64-byte run at once
                        const int g = (i + a_c) & (GROUP - 1);
                        const int mine = g == 0 ? tot[0] : g == 1 ? tot[1] : g == 2 ? tot[2] : tot[3];
                        __hip_atomic_fetch_add(reinterpret_cast<int*>(xblock(xt, 0, kXbOacc)) + (a_h * GROUP + g) * kHd + d, mine + L.osum[g][d],
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            } else {
                __builtin_amdgcn_s_sleep(56);
                for (int i = 0; i < min(nchunks, 8); i++) __builtin_amdgcn_s_sleep(5);
                gu_slice(2);
            }
            stamp();
            bar.arrive(!is_s);
        }

        // ================= phase 4: attention dequant + quant -> o_proj rows (8 per workgroup, 2 per wave 0..3) + residual =================
        {
            i32x4 wr[2][2];
            float wsc[2] = {0.0f, 0.0f}, wsm[2] = {0.0f, 0.0f};
            if (!is_s) {
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    if constexpr (W4) {
                        i32x4 one[1];
                        mega_load_rows<1>(w.wo, H / 2, wg * 8 + wave + 4 * j, lane, one);
                        wr[j][0] = one[0];
                        wsm[j] = ldc_f(w.mo + wg * 8 + wave + 4 * j);
                    } else {
                        mega_load_rows<2>(w.wo, H, wg * 8 + wave + 4 * j, lane, wr[j]);
                    }
                    wsc[j] = ldc_f(w.so + wg * 8 + wave + 4 * j);
                }
            }
            const float osa = a_s[t >> 4], osv = v_s[t >> 6];         // elements 4t..4t+3 lie in query head t/16
            // the stream waves' previous slice has landed long ago, so they can share the activation loads
            float v[4], xr[2] = {0.0f, 0.0f};
            bar.wait();
            stamp();
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const unsigned long long w2 = ld_u64(reinterpret_cast<const unsigned long long*>(reinterpret_cast<const int*>(xblock(xt, 0, kXbOacc)) + 4 * t + 2 * i));
                v[2 * i] = (float)(int)(unsigned)w2 * osa * osv;
                v[2 * i + 1] = (float)(int)(unsigned)(w2 >> 32) * osa * osv;
            }
            if (!is_s && lane == 0) {                                 // residual inputs, fetched with the activations
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int row = wg * 8 + wave + 4 * j;
                    if (l == 0) xr[j] = p.x_in ? p.x_in[row] : __half2float(p.embed[(size_t)tok * H + row]);
                    else xr[j] = L.res8[wave + 4 * j];              // this workgroup's own rows of x, left there by phase 6

                }
            }
            const float4 z4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            float sx, bx = 0.0f;
            if constexpr (W4) { const float2 sb = norm_quant_2048_u4(v, z4, false, p.eps, L, [&]() { gu_slice(3); }); sx = sb.x; bx = sb.y; }
            else sx = norm_quant_2048(v, z4, false, p.eps, L, [&]() { gu_slice(3); });
            if (!is_s) {
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    if constexpr (W4) {
                        const i32x4 one[1] = {wr[j][0]};
                        float out = (float)mega_dot_row4<1>(one, L.xq, lane) * sx * wsc[j];
                        out = out + bx * wsm[j];
                        if (lane == 0) L.res8[wave + 4 * j] = out + xr[j];
                    } else {
                        const int a0 = mega_dot_row<2>(wr[j], L.xq, lane);
                        if (lane == 0) L.res8[wave + 4 * j] = (float)a0 * sx * wsc[j] + xr[j];
                    }
                }
            }
            // the workgroup's eight outputs leave as one 32-byte store: eight single-lane stores from four waves into
            // the same sector take longer to be acknowledged, and the barrier waits for that
            __syncthreads();
            publish8(kXbX2, L.res8, tag);
            stamp();
            // no grid barrier: the consumers poll the tagged words
        }

        // ================= phase 5: RMSNorm + quant -> gate/up rows (64 per workgroup, 16 per stream wave) + SiLU*up =================
        {
            // Stream wave s holds rows 0..7 of its 16 gate/up rows in registers and rows 8..15 in LDS; it multiplies the
            // first eight itself, wave s (of waves 0..3) the other eight.  After the folding below lane L holds the sum
            // of row ridx of its wave's eight.
            const int ridx = 4 * (lane & 1) + 2 * ((lane >> 1) & 1) + ((lane >> 2) & 1);
            const int ow = wave & 3, half = is_s ? 0 : 8;
            const float gsc = w.sgu[wg * 64 + ow * 16 + half + ridx]; // read before this phase's prefetch is issued
            // W4A4: a stream wave multiplies all 16 of its rows (rows ridx and 8 + ridx per lane after the folding)
            float gsc_b = 0.0f, gsm_a = 0.0f, gsm_b = 0.0f;
            if constexpr (W4) {
                gsc_b = w.sgu[wg * 64 + ow * 16 + 8 + ridx];
                gsm_a = w.mgu[wg * 64 + ow * 16 + ridx];
                gsm_b = w.mgu[wg * 64 + ow * 16 + 8 + ridx];
            }
            const float4 gam = reinterpret_cast<const float4*>(g1)[t];
            float v[4];
            poll_tagged4(my_copy(kXbX2), tag, bar.err, L.f + (t >> 6) * 256, v);
            stamp();
            auto down_row_0 = [&]() {
                // Runs after the first workgroup barrier of the reduction below, i.e. once ALL eight waves have their
                // share of x2: every workgroup has then published x2, so every workgroup has read the accumulators,
                // and this workgroup's eight can be cleared.  (A wave's own poll only covers the 256 words of 32
                // producers: clearing right behind it wiped accumulators that a slower workgroup had yet to read.)
                // The next parts are added a layer later, by workgroups that have polled this workgroup's x, which
                // the same threads store after this store has been acknowledged.
                if (t < 8) st_i(reinterpret_cast<int*>(xblock(xt, 0, kXbOacc)) + wg * 8 + t, 0);
                __builtin_amdgcn_s_waitcnt(0x0F70);                   // vmcnt(0): see gu_slice
                if (is_s) {
                    if constexpr (W4) mega_row4_to_lds(w.wd, wg * 8 + sw * 2, lane, L.wd[sw * 2]);
                    else mega_row_to_lds(w.wd, wg * 8 + sw * 2, lane, L.wd[sw * 2]);
                }
            };
            float sx, bx = 0.0f;
            if constexpr (W4) { const float2 sb = norm_quant_2048_u4(v, gam, true, p.eps, L, down_row_0); sx = sb.x; bx = sb.y; }
            else sx = norm_quant_2048(v, gam, true, p.eps, L, down_row_0);
            if (l == 1) fine();
            // eight per-lane partial sums folded with a transposing butterfly: each step halves the number of live
            // values, so 7 + 3 cross-lane exchanges replace 8 x 6.  Afterwards lane L holds the complete sum of row
            // 4*(L&1) + 2*(L>>1 & 1) + (L>>2 & 1).
            auto fold8 = [&](const int (&part)[8]) {
                int q4[4], q2[2];
                {
                    const bool hi = lane & 1;
#pragma unroll
                    for (int i = 0; i < 4; i++) q4[i] = (hi ? part[i + 4] : part[i]) + lane_xor_i<1>(hi ? part[i] : part[i + 4]);
                }
                {
                    const bool hi = lane & 2;
#pragma unroll
                    for (int i = 0; i < 2; i++) q2[i] = (hi ? q4[i + 2] : q4[i]) + lane_xor_i<2>(hi ? q4[i] : q4[i + 2]);
                }
                int sum;
                {
                    const bool hi = lane & 4;
                    sum = (hi ? q2[1] : q2[0]) + lane_xor_i<4>(hi ? q2[0] : q2[1]);
                }
                sum += lane_xor_i<8>(sum);
                sum += lane_xor_i<16>(sum);
                sum += lane_xor_i<32>(sum);
                return sum;
            };
            if constexpr (W4) {
                if (is_s) {
                    const i32x4 ones = {0x11111111, 0x11111111, 0x11111111, 0x11111111};
                    i32x4 xs = reinterpret_cast<const i32x4*>(L.xq)[lane];
                    xs.x ^= 0x88888888; xs.y ^= 0x88888888; xs.z ^= 0x88888888; xs.w ^= 0x88888888;   // a -> a - 8
                    int part_a[8], part_b[8];
#pragma unroll
                    for (int r = 0; r < 8; r++) {
                        const i32x4 wa = gu[r >> 1][r & 1], wb = gu[(8 + r) >> 1][r & 1];
                        part_a[r] = dot32_i4(wa, xs, 0) + 8 * dot32_i4(wa, ones, 0);
                        part_b[r] = dot32_i4(wb, xs, 0) + 8 * dot32_i4(wb, ones, 0);
                    }
                    const int sum_a = fold8(part_a), sum_b = fold8(part_b);
                    float mine_a = (float)sum_a * sx * gsc;
                    mine_a = mine_a + bx * gsm_a;
                    float mine_b = (float)sum_b * sx * gsc_b;
                    mine_b = mine_b + bx * gsm_b;
                    const float other_a = lane_xor_f<4>(mine_a), other_b = lane_xor_f<4>(mine_b);   // row ridx^1: the other half of the SwiGLU pair
                    if (lane < 4) {                                // lanes 0..3 hold the (even) gate rows
                        L.hst[ow * 8 + (ridx >> 1)] = other_a * silu_f(mine_a);
                        L.hst[ow * 8 + 4 + (ridx >> 1)] = other_b * silu_f(mine_b);
                    }
                }
            } else {
                int part[8];
                {
                    const i32x4 x0 = reinterpret_cast<const i32x4*>(L.xq)[lane], x1 = reinterpret_cast<const i32x4*>(L.xq)[lane + 64];
                    if (is_s) {
#pragma unroll
                        for (int r = 0; r < 8; r++) part[r] = dot16(gu[r][1], x1, dot16(gu[r][0], x0, 0));
                    } else {
                        // rows 8..15 from LDS (complete and visible: their stream wave waited for them at the head of
                        // this phase's prefetch hook, before the barrier that ended the quantisation)
                        const i32x4* g2 = reinterpret_cast<const i32x4*>(L.gu2[ow]);
                        const i32x4* g3 = reinterpret_cast<const i32x4*>(L.wd[ow * 2 + 1]);
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            part[r] = dot16(g2[lane + 64 * (2 * r + 1)], x1, dot16(g2[lane + 64 * (2 * r)], x0, 0));
                            part[4 + r] = dot16(g3[lane + 64 * (2 * r + 1)], x1, dot16(g3[lane + 64 * (2 * r)], x0, 0));
                        }
                    }
                }
                const int sum = fold8(part);
                const float mine = (float)sum * sx * gsc;
                const float other = lane_xor_f<4>(mine);           // row ridx^1: the other half of the SwiGLU pair
                if (lane < 4) L.hst[ow * 8 + (half >> 1) + (ridx >> 1)] = other * silu_f(mine);   // lanes 0..3 hold the (even) gate rows
            }
            __syncthreads();
            if (l == 1) fine();
            if (t < 64) {
                // This workgroup's 32 values are the indices 32*wg .. 32*wg+31 of the 8192-vector: the first four stages
                // of the transform (index bits 1..4, in that order) pair elements inside the block, so wave 0 does them
                // here once instead of every workgroup doing them on the whole vector in phase 6.
                float hv = L.hst[t & 31];
                hv = lane_butterfly_s<2>(hv, lane_sign<2>(t));
                hv = lane_butterfly_s<4>(hv, lane_sign<4>(t));
                hv = lane_butterfly_s<8>(hv, lane_sign<8>(t));
                hv = lane_butterfly_s<16>(hv, lane_sign<16>(t));
                if (t < 32) st_f(&hbuf[wg * 32 + t], hv);             // stored by a wave with no prefetch in flight
            }
            if (l == 1) fine();
            stamp();
            bar.arrive(!is_s);
        }

        // ================= phase 6: Hadamard R4 + quant -> down rows (8 per workgroup, one per wave) + residual =================
        {
            // Each wave multiplies one of the eight rows: stream wave s the even row 2s, wave s (of 0..3) the odd row 2s+1
            // that stream wave s fetched into LDS.
            const int drow = wg * 8 + (wave & 3) * 2 + (is_s ? 0 : 1);
            const float dsc = ldc_f(w.sd + drow);
            float dsm = 0.0f;
            if constexpr (W4) dsm = ldc_f(w.md + drow);
            float xres = 0.0f;
            bar.wait();
            stamp();
            if (lane == 0) xres = L.res8[drow - wg * 8];              // this workgroup's own rows of x2, left there by phase 4
            // 8192-point transform on all 512 threads, stage order bits 1,2,...,12,0 (bit-exact order, see
            // fht_kernels.h).  Every remaining stage is a butterfly between registers of one thread, with two passes
            // through LDS between the three layouts:
            //   A: i = (t>>3)*128 + j*32 + (t&7)*4 + e -> stages 1..4 came done from phase 5; here 5 and 6 (j)
            //   B: i = (t>>7)*2048 + r*128 + (t&127)   -> stages 7..10 (r)
            //   C: i = q*2048 + 4t + e                 -> stages 11 and 12 (q), then 0 (e)
            float4 a[4];
            const int abase = (t >> 3) * 128 + (t & 7) * 4;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                a[j] = *reinterpret_cast<const float4*>(hbuf + abase + j * 32);   // ordinary loads: they may hit in L2
            }
            __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0): the h loads are complete
            if (is_s) {
                if constexpr (W4) mega_row4_to_lds(w.wd, wg * 8 + sw * 2 + 1, lane, L.wd[sw * 2 + 1]);
                else mega_row_to_lds(w.wd, wg * 8 + sw * 2 + 1, lane, L.wd[sw * 2 + 1]);
            }
            if (l == 1) fine();
#pragma unroll
            for (int bit = 1; bit < 4; bit <<= 1)                                                                       // bits 5, 6
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if ((j & bit) == 0) {
                        const float4 u = a[j], v = a[j | bit];
                        a[j] = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
                        a[j | bit] = make_float4(u.x - v.x, u.y - v.y, u.z - v.z, u.w - v.w);
                    }
            if (l == 1) fine();
#pragma unroll
            for (int j = 0; j < 4; j++) reinterpret_cast<float4*>(L.f)[(abase >> 2) + j * 8] = a[j];
            __syncthreads();
            if (l == 1) fine();
            float b[16];
            const int bbase = (t >> 7) * 2048 + (t & 127);
#pragma unroll
            for (int r = 0; r < 16; r++) b[r] = L.f[bbase + r * 128];
#pragma unroll
            for (int bit = 1; bit < 16; bit <<= 1)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    if ((r & bit) == 0) { const float u = b[r], v = b[r | bit]; b[r] = u + v; b[r | bit] = u - v; }
            // each thread re-writes exactly the slots it read, so no barrier is needed before this store
#pragma unroll
            for (int r = 0; r < 16; r++) L.f[bbase + r * 128] = b[r];
            __syncthreads();
            // last pass (i = q*2048 + 4t + e): bit 11 pairs q with q^1, bit 12 q with q^2, bit 0 pairs e with e^1, all
            // inside the thread, and the quantised bytes of a thread are four consecutive ones per q
            float4 c4[4];
#pragma unroll
            for (int q = 0; q < 4; q++) c4[q] = reinterpret_cast<const float4*>(L.f)[q * 512 + t];
#pragma unroll
            for (int q = 0; q < 4; q += 2) {                                                                          // bit 11
                const float4 u = c4[q], v = c4[q + 1];
                c4[q] = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
                c4[q + 1] = make_float4(u.x - v.x, u.y - v.y, u.z - v.z, u.w - v.w);
            }
#pragma unroll
            for (int q = 0; q < 2; q++) {                                                                             // bit 12
                const float4 u = c4[q], v = c4[q + 2];
                c4[q] = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
                c4[q + 2] = make_float4(u.x - v.x, u.y - v.y, u.z - v.z, u.w - v.w);
            }
            if (l == 1) fine();
            float amax = 0.0f;
            float b2[16];
#pragma unroll
            for (int q = 0; q < 4; q++) {                                                                             // bit 0
                b2[4 * q + 0] = c4[q].x + c4[q].y;
                b2[4 * q + 1] = c4[q].x - c4[q].y;
                b2[4 * q + 2] = c4[q].z + c4[q].w;
                b2[4 * q + 3] = c4[q].z - c4[q].w;
            }
#pragma unroll
            for (int r = 0; r < 16; r++) amax = fmaxf(amax, fabsf(b2[r]));
            // division by the transform's scale as in fht_kernels.h: reciprocal + exact residual step, plain division
            // outside the safe range; the largest quotient is the quotient of the largest magnitude
            if (div_fast_ok(amax, p.fht_scale)) {
                const float rs = 1.0f / p.fht_scale;
#pragma unroll
                for (int r = 0; r < 16; r++) b2[r] = div_fast(b2[r], p.fht_scale, rs);
            } else {
#pragma unroll
                for (int r = 0; r < 16; r++) b2[r] = b2[r] / p.fht_scale;
            }
            amax = amax / p.fht_scale;
            if (l == 1) fine();
            float sx, bx = 0.0f;
            if constexpr (W4) {
                // asymmetric uint4: largest and smallest of the scaled values (the thread's own 16, then the workgroup's)
                float vmax = b2[0], vmin = b2[0];
#pragma unroll
                for (int r = 1; r < 16; r++) { vmax = fmaxf(vmax, b2[r]); vmin = fminf(vmin, b2[r]); }
                vmax = mega_block_max_h(vmax, L.red_max, NoHook());
                vmin = mega_block_min_h(vmin, L.red_min, NoHook());
                sx = (vmax - vmin) / 15.0f;
                if (sx == 0.0f) sx = 1.0f;
                bx = vmin;
                uint16_t w16[4];
                quant_u4_pack(b2, vmin, sx, w16);
#pragma unroll
                for (int q = 0; q < 4; q++) reinterpret_cast<uint16_t*>(L.xq)[q * 512 + t] = w16[q];   // nibble q*2048 + 4t + e
            } else {
                amax = mega_block_max_h(amax, L.red_max, NoHook());
                sx = sym_scale_127_uniform(amax);
                if (l == 1) fine();
                int n16[16];
                quant_vector(b2, sx, n16);
#pragma unroll
                for (int q = 0; q < 4; q++)
                    reinterpret_cast<uint32_t*>(L.xq)[q * 512 + t] = pack4_i8(n16[4 * q], n16[4 * q + 1], n16[4 * q + 2], n16[4 * q + 3]);
            }
            if (is_s) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): both down rows of this stream wave have landed in LDS
            __syncthreads();                               // ... and are visible to the wave that multiplies the odd one
            if (l == 1) fine();
            if constexpr (W4) {
                float out = (float)mega_dot_row4_lds(L.wd[(wave & 3) * 2 + (is_s ? 0 : 1)], L.xq, lane) * sx * dsc;
                out = out + bx * dsm;
                if (lane == 0) L.res8[drow - wg * 8] = out + xres;
            } else {
                const int a0 = mega_dot_row_lds(L.wd[(wave & 3) * 2 + (is_s ? 0 : 1)], L.xq, lane);
                if (lane == 0) L.res8[drow - wg * 8] = (float)a0 * sx * dsc + xres;
            }
            __syncthreads();
            if (t < 16) {
                __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0): the accumulator reset of phase 5 has landed
                publish8(kXbX, L.res8, tag);                      // one 64-byte store per copy, as in phase 4
                if (t < 8 && l == p.n_layers - 1) st_f(&p.x[wg * 8 + t], L.res8[t]);   // the hidden state the host reads back
            }
            if (l == 1) fine();
            if (l == 1) fine();
            stamp();
        }
    }

    // ================= head: final RMSNorm -> lm_head rows, per-workgroup argmax candidate =================
    if (p.want_head) {
        int t_head = threadIdx.x;                 // opaque copy, as in the layer loop: nothing per-thread stays live across it
        asm volatile("" : "+v"(t_head));
        const int t = t_head, lane = t & 63;
        const int rows_per_wg = (p.vocab + kMegaWG - 1) / kMegaWG;
        const int row_begin = wg * rows_per_wg, row_end = min(p.vocab, row_begin + rows_per_wg);
        constexpr int U = 4;
        int r = row_begin + wave;
        float best = -INFINITY;
        int bi = 0x7fffffff;
        auto keep_logit = [&](float s, int row) {              // one finished row: wave-uniform s
            if (row < row_end) {
                if (lane == 0) {
                    p.logits[row] = s;
                    if (sampling) L.f[4096 + (row - row_begin)] = s;      // L.f[0..2047] holds the normalised vector
                }
                if (s > best || (s == best && row < bi)) { best = s; bi = row; }
            }
        };
        if constexpr (W4) {
            // int4 output head: rows of 1024 bytes against the normalised vector quantised to asymmetric uint4
            i32x4 wv[U][1];
            auto load_group = [&](int rr) {
#pragma unroll
                for (int u = 0; u < U; u++)
                    mega_load_rows<1>(reinterpret_cast<const int8_t*>(p.head_w4), H / 2, min(rr + u * kMegaWaves, p.vocab - 1), lane, wv[u]);
            };
            load_group(r);
            float v[4];
            poll_tagged4(my_copy(kXbX), seq0 + (unsigned)((step + 1) * p.n_layers), bar.err, L.f + (t >> 6) * 256, v);
            stamp();
            const float4 g = reinterpret_cast<const float4*>(p.gamma + (size_t)(2 * p.n_layers) * H)[t];
            const float2 sb = norm_quant_2048_u4(v, g, true, p.eps, L, NoHook());
            for (; r < row_end; r += U * kMegaWaves) {
                int acc[U];
#pragma unroll
                for (int u = 0; u < U; u++) acc[u] = mega_dot_row4<1>(wv[u], L.xq, lane);
                const int rn = r + U * kMegaWaves;
                if (rn < row_end) load_group(rn);
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const int row = min(r + u * kMegaWaves, p.vocab - 1);
                    float s = (float)acc[u] * sb.x * p.head_s[row];
                    s = s + sb.y * p.head_sum[row];
                    keep_logit(s, r + u * kMegaWaves);
                }
            }
        } else {
        using h16x8 = _Float16 __attribute__((ext_vector_type(8)));
        const h16x8* table = reinterpret_cast<const h16x8*>(p.embed);
        h16x8 wv[U][4];
        auto load_group = [&](int r) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int row = min(r + u * kMegaWaves, p.vocab - 1);
#pragma unroll
                for (int i = 0; i < 4; i++) wv[u][i] = __builtin_nontemporal_load(table + (size_t)row * (H / 8) + lane + 64 * i);
            }
        };
        load_group(r);
        float v[4];
        poll_tagged4(my_copy(kXbX), seq0 + (unsigned)((step + 1) * p.n_layers), bar.err, L.f + (t >> 6) * 256, v);
        stamp();
        float ss = (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
        ss = block_sum<kMegaWaves>(ss, L.red);
        const float rms = 1.0f / sqrtf(ss / 2048.0f + p.eps);
        const float4 g = reinterpret_cast<const float4*>(p.gamma + (size_t)(2 * p.n_layers) * H)[t];
        reinterpret_cast<float4*>(L.f)[t] = make_float4(v[0] * rms * g.x, v[1] * rms * g.y, v[2] * rms * g.z, v[3] * rms * g.w);
        __syncthreads();
        float nv[4][8];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int e = 0; e < 8; e++) nv[i][e] = L.f[(lane + 64 * i) * 8 + e];
        for (; r < row_end; r += U * kMegaWaves) {
            float acc[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                acc[u] = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[u] += (float)wv[u][i][e] * nv[i][e];
            }
            const int rn = r + U * kMegaWaves;
            if (rn < row_end) load_group(rn);
#pragma unroll
            for (int u = 0; u < U; u++) keep_logit(wave_sum(acc[u]), r + u * kMegaWaves);
        }
        }
        if (lane == 0) { L.bestv[wave] = best; L.besti[wave] = bi; }
        __syncthreads();
        if (t == 0) {
            for (int i = 1; i < kMegaWaves; i++)
                if (L.bestv[i] > best || (L.bestv[i] == best && L.besti[i] < bi)) { best = L.bestv[i]; bi = L.besti[i]; }
            st_f(&p.am_v[wg], best);
            st_i(&p.am_i[wg], bi);
        }
        stamp();
        if (sampling) {
            // Top-k sampling (Modules/Logits.h:145-279) without leaving the kernel: this workgroup's top_k logits ->
            // grid barrier -> every workgroup selects the global top_k among the kMegaWG * top_k candidates and draws
            // the same token from them (same inputs, same arithmetic), so the next step needs no further exchange.
            float val[kTopKMax];
            int idx[kTopKMax];
#pragma unroll
            for (int k = 0; k < kTopKMax; k++) { val[k] = -1e32f; idx[k] = 0x7fffffff; }
            for (int i = t; i < row_end - row_begin; i += kMegaT) topk_insert(val, idx, p.top_k, L.f[4096 + i], row_begin + i);
            topk_block_select<kMegaT>(val, idx, p.top_k, L.tk_val, L.tk_idx);
            if (t < p.top_k) { st_f(&p.cand_v[wg * kTopKMax + t], L.tk_val[t]); st_i(&p.cand_i[wg * kTopKMax + t], L.tk_idx[t]); }
            bar.arrive();
            bar.wait();
#pragma unroll
            for (int k = 0; k < kTopKMax; k++) { val[k] = -1e32f; idx[k] = 0x7fffffff; }
            for (int i = t; i < kMegaWG * p.top_k; i += kMegaT) {
                const int slot = (i / p.top_k) * kTopKMax + i % p.top_k;
                topk_insert(val, idx, p.top_k, ld_f(&p.cand_v[slot]), ld_i(&p.cand_i[slot]));
            }
            topk_block_select<kMegaT>(val, idx, p.top_k, L.tk_val, L.tk_idx);
            if (t == 0) {
                float prob[kTopKMax];
                const int sel = topk_sample_rank(L.tk_val, p.top_k, p.rands[step_base + step], 1, prob);
                const int chosen = L.tk_idx[sel];
                L.tk_tok = (unsigned)chosen < (unsigned)p.vocab ? chosen : 0;   // after a time-out the candidates may be anything
                L.stop = bar.dead || ld_i(bar.err) == 1;
            }
            __syncthreads();
            tok = __builtin_amdgcn_readfirstlane(L.tk_tok);
            stop = __builtin_amdgcn_readfirstlane(L.stop);
            if (wg == 0 && t == 0) p.tokens_out[step_base + step] = tok;
            __syncthreads();                                        // L.tk_* and L.f are reused by the next step
        } else if (greedy) {
            // every workgroup picks the winner among the kMegaWG candidates (largest value, then smallest index)
            bar.arrive();
            bar.wait();
            float cv = -INFINITY;
            int ci = 0x7fffffff;
            if (t < kMegaWG) { cv = ld_f(&p.am_v[t]); ci = ld_i(&p.am_i[t]); }
            if (t == 0) L.stop = bar.dead || ld_i(bar.err) == 1;   // fetched along with the candidates
#pragma unroll
            for (int m = 1; m < 64; m <<= 1) {
                const float ov = __shfl_xor(cv, m);
                const int oi = __shfl_xor(ci, m);
                if (ov > cv || (ov == cv && oi < ci)) { cv = ov; ci = oi; }
            }
            if (lane == 0) { L.bestv[t >> 6] = cv; L.besti[t >> 6] = ci; }
            __syncthreads();
            cv = L.bestv[0]; ci = L.besti[0];
#pragma unroll
            for (int i = 1; i < kMegaWG / 64; i++)
                if (L.bestv[i] > cv || (L.bestv[i] == cv && L.besti[i] < ci)) { cv = L.bestv[i]; ci = L.besti[i]; }
            tok = __builtin_amdgcn_readfirstlane((unsigned)ci < (unsigned)p.vocab ? ci : 0);   // after a time-out the candidates may be anything
            stop = __builtin_amdgcn_readfirstlane(L.stop);
            if (wg == 0 && t == 0) p.tokens_out[step_base + step] = tok;
            __syncthreads();                                        // L.bestv/besti are reused by the next step
        }
    }
    steps_done = step + 1;
    }   // step loop (left early only after a barrier time-out, which the error flag reports)
    if (wg == 0 && is_t0()) {
        p.state[2] = (int)bar.epoch;
        p.state[4] = (int)(seq0 + (unsigned)(steps_done * p.n_layers));
        if (greedy) { p.token[0] = tok; p.state[0] = pos0 + steps_done; p.state[1] = step_base + steps_done; }
    }
#ifdef FX_MEGA_FINE_STAMPS
    if (p.timeline && is_t0()) p.timeline[p.n_layers * 12 + 2 + 64 + kMegaWG + wg] = wall_clock64();     // workgroup exit
#endif
}

__global__ __launch_bounds__(kMegaT, 1) void decode_mega_kernel(MegaParams p) { decode_mega_body<false>(p); }
__global__ __launch_bounds__(kMegaT, 1) void decode_mega_w4_kernel(MegaParams p) { decode_mega_body<true>(p); }

}  // namespace fx

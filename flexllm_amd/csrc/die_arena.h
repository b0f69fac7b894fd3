// Memory for the words that workgroups hand to each other inside a launch, sorted by the I/O die it is attached to.
//
// The chip is two I/O dies with four XCDs and half of the HBM stacks each.  A coherent (past-L2) store or load from an
// XCD to memory behind the other die crosses the die-to-die link: an exchange of one word among the 32 workgroups of an
// XCD takes 0.9 us through memory of its own die and 1.1-1.9 us through the other die's (measured: the calibration
// below).  Physical memory alternates between the dies in blocks of 8 KiB, in a pattern that depends on higher address
// bits, so which die a block belongs to is MEASURED here, once, when a model is created.
//
// Users keep every exchanged array in two copies, one per die: the producer stores into both (a store is posted, its
// trip across the link is nobody's wait), the consumer polls the copy of its own die.  Correctness never depends on
// the outcome of the calibration - both copies always hold the same words - only the speed does.  When the
// calibration fails (placement of workgroups not round-robin over eight XCDs, a wait timed out, no clear difference)
// take_pair() hands out one block for both copies and the users degrade to a single copy.
#pragma once
#include "common.h"
#include <vector>

namespace fx {

constexpr size_t kDieBlock = 8192;        // bytes: the granularity at which memory alternates between the dies
constexpr int kDieProbeWG = 256;          // workgroups of the calibration kernel: 32 per XCD on a chip of 8 XCDs
constexpr int kDieProbeWarm = 8, kDieProbeRounds = 32;

// Workgroup w belongs to group w % 8 (the XCD it runs on when workgroups are dealt round-robin).  Per round every
// workgroup stores one tagged word into the block and polls the 32 words of its group, past L2 both ways.
// out[b][w] = wall-clock ticks (100 MHz) of the timed rounds, xcc[w] = the XCD the workgroup really ran on.
static __global__ __launch_bounds__(64) void die_probe_kernel(unsigned long long* block, long long* out, unsigned* xcc, int* err) {
    const int wg = blockIdx.x, group = wg % 8, rank = wg / 8, lane = threadIdx.x;
    if (lane == 0) {
        unsigned x;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
        xcc[wg] = x & 15u;
    }
    unsigned long long* base = block + group * 64;
    long long t0 = 0;
    bool dead = false;
    for (int r = 1; r <= kDieProbeWarm + kDieProbeRounds && !dead; r++) {
        if (r == kDieProbeWarm + 1) t0 = wall_clock64();
        if (lane == 0) __hip_atomic_store(&base[rank], ((unsigned long long)r << 32) | (unsigned)rank, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (lane < 32) {
            int it = 0;
            for (;;) {
                const unsigned long long w = __hip_atomic_load(&base[lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const bool ok = (int)((unsigned)(w >> 32) - (unsigned)r) >= 0;
                if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
                if (++it > (1 << 14) || ((it & 63) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                    __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);      // bounded: give up, everybody follows
                    dead = true;
                    break;
                }
            }
        }
        dead = __builtin_amdgcn_ballot_w64(dead) != 0;
    }
    if (lane == 0) out[wg] = wall_clock64() - t0;
}

// Pure host arithmetic of the calibration.  us[b * 8 + x] = exchange round of XCD x's workgroups through block b.
// XCDs of one die see the same blocks as near, so the sign of the correlation with XCD 0 over the blocks splits them
// into the two dies (*die_mask: bit x = die of XCD x, XCD 0 on die 0); a block belongs to the die whose four XCDs are at
// least 4 % faster on average (die_of_block[b] = 0 or 1), otherwise to none (-1).  Returns false - no usable picture -
// unless each die has exactly four XCDs and at least four blocks.
static bool die_classify(const float* us, int n_blocks, unsigned* die_mask, int* die_of_block, float* near_us, float* far_us) {
    if (n_blocks < 8) return false;
    double mean[8] = {0};
    for (int b = 0; b < n_blocks; b++)
        for (int x = 0; x < 8; x++) mean[x] += us[(size_t)b * 8 + x] / n_blocks;
    unsigned mask = 0;
    int on_die1 = 0;
    for (int x = 1; x < 8; x++) {
        double c = 0.0;
        for (int b = 0; b < n_blocks; b++) c += (us[(size_t)b * 8] - mean[0]) * (us[(size_t)b * 8 + x] - mean[x]);
        if (c < 0.0) { mask |= 1u << x; on_die1++; }
    }
    if (on_die1 != 4) return false;
    double near_sum = 0.0, far_sum = 0.0;
    int count[2] = {0, 0};
    for (int b = 0; b < n_blocks; b++) {
        double s[2] = {0.0, 0.0};
        for (int x = 0; x < 8; x++) s[(mask >> x) & 1] += us[(size_t)b * 8 + x] / 4.0;
        const int die = s[0] < s[1] ? 0 : 1;
        if (!(s[1 - die] >= 1.04 * s[die])) { die_of_block[b] = -1; continue; }     // no clear difference (or not a number)
        die_of_block[b] = die;
        count[die]++;
        near_sum += s[die];
        far_sum += s[1 - die];
    }
    if (count[0] < 4 || count[1] < 4) return false;
    *die_mask = mask;
    *near_us = (float)(near_sum / (count[0] + count[1]));
    *far_us = (float)(far_sum / (count[0] + count[1]));
    return true;
}

struct DieArena {
    char* base = nullptr;                  // 8 KiB aligned
    int n_blocks = 0;
    bool calibrated = false;
    unsigned die_mask = 0xF0;              // bit x = the die of XCD x
    std::vector<int> blocks[2];            // calibrated: the blocks attached to die 0 / die 1, not yet handed out
    int next_plain = 0;                    // not calibrated: the next block
    float near_us = 0.0f, far_us = 0.0f;   // calibrated: mean exchange round through own-die / other-die memory

    // Two blocks, a[0] attached to die 0 and a[1] to die 1 (or one block for both when that is not known), filled with
    // `fill` bytes.  Returns false when the arena is used up.
    bool take_pair(void* (&a)[2], int fill) {
        if (calibrated) {
            if (blocks[0].empty() || blocks[1].empty()) return false;
            a[0] = base + (size_t)blocks[0].back() * kDieBlock; blocks[0].pop_back();
            a[1] = base + (size_t)blocks[1].back() * kDieBlock; blocks[1].pop_back();
        } else {
            if (next_plain >= n_blocks) return false;
            a[0] = a[1] = base + (size_t)next_plain++ * kDieBlock;
        }
        return hipMemset(a[0], fill, kDieBlock) == hipSuccess && hipMemset(a[1], fill, kDieBlock) == hipSuccess;
    }
};

// Allocates n_blocks blocks (`raw` receives the pointer to free) and measures which die each belongs to.
// want_calibration == false skips the measurement (single-copy operation).
static int die_arena_create(DieArena& a, int n_blocks, bool want_calibration, void** raw) {
    a = DieArena();
    FX_REQUIRE(n_blocks >= 8 && n_blocks <= 255, "die arena: %d blocks (users keep block indices in a byte)", n_blocks);
    FX_HIP(hipMalloc(raw, (size_t)(n_blocks + 1) * kDieBlock));
    a.base = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(*raw) + kDieBlock - 1) & ~(uintptr_t)(kDieBlock - 1));
    a.n_blocks = n_blocks;
    FX_HIP(hipMemset(a.base, 0, (size_t)n_blocks * kDieBlock));
    int cus = 0, dev = 0;
    FX_HIP(hipGetDevice(&dev));
    FX_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (!want_calibration || cus < kDieProbeWG) return FLEXLLM_OK;

    long long* d_out = nullptr;
    unsigned* d_xcc = nullptr;
    int* d_err = nullptr;
    FX_HIP(hipMalloc((void**)&d_out, sizeof(long long) * kDieProbeWG * n_blocks));
    auto cleanup = [&]() { (void)hipFree(d_out); (void)hipFree(d_xcc); (void)hipFree(d_err); };
    if (hipMalloc((void**)&d_xcc, sizeof(unsigned) * kDieProbeWG) != hipSuccess || hipMalloc((void**)&d_err, sizeof(int)) != hipSuccess ||
        hipMemset(d_err, 0, sizeof(int)) != hipSuccess) {
        cleanup();
        set_error("die arena: allocation of the calibration buffers failed");
        return FLEXLLM_EHIP;
    }
    for (int b = 0; b < n_blocks; b++)
        die_probe_kernel<<<kDieProbeWG, 64>>>(reinterpret_cast<unsigned long long*>(a.base + (size_t)b * kDieBlock),
                                             d_out + (size_t)b * kDieProbeWG, d_xcc, d_err);
    std::vector<long long> out((size_t)kDieProbeWG * n_blocks);
    std::vector<unsigned> xcc(kDieProbeWG);
    int err = 0;
    const bool ok = hipDeviceSynchronize() == hipSuccess &&
                    hipMemcpy(out.data(), d_out, sizeof(long long) * out.size(), hipMemcpyDeviceToHost) == hipSuccess &&
                    hipMemcpy(xcc.data(), d_xcc, sizeof(unsigned) * kDieProbeWG, hipMemcpyDeviceToHost) == hipSuccess &&
                    hipMemcpy(&err, d_err, sizeof(int), hipMemcpyDeviceToHost) == hipSuccess &&
                    hipMemset(a.base, 0, (size_t)n_blocks * kDieBlock) == hipSuccess;
    cleanup();
    if (!ok) { set_error("die arena: the calibration run failed: %s", hipGetErrorString(hipGetLastError())); return FLEXLLM_EHIP; }
    if (err) return FLEXLLM_OK;                                     // a wait timed out: single copy
    for (int w = 0; w < kDieProbeWG; w++)
        if (xcc[w] != (unsigned)(w % 8)) return FLEXLLM_OK;         // not eight XCDs dealt round-robin: single copy

    // t[b][x]: the slowest workgroup of XCD x, microseconds per round
    std::vector<float> t((size_t)n_blocks * 8, 0.0f);
    for (int b = 0; b < n_blocks; b++)
        for (int w = 0; w < kDieProbeWG; w++) {
            const float us = (float)out[(size_t)b * kDieProbeWG + w] / 100.0f / kDieProbeRounds;
            float& slot = t[(size_t)b * 8 + w % 8];
            slot = us > slot ? us : slot;
        }
    std::vector<int> die_of(n_blocks);
    unsigned mask = 0;
    if (!die_classify(t.data(), n_blocks, &mask, die_of.data(), &a.near_us, &a.far_us)) return FLEXLLM_OK;   // no clear picture: single copy
    for (int b = 0; b < n_blocks; b++)
        if (die_of[b] >= 0) a.blocks[die_of[b]].push_back(b);
    a.die_mask = mask;
    a.calibrated = true;
    return FLEXLLM_OK;
}

}  // namespace fx

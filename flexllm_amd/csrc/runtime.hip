// Error plumbing, thin runtime helpers for FFI hosts, and the counter-based fill kernels.
#include "common.h"
#include <hip/hip_fp16.h>
#include <map>
#include <mutex>
#include <stdarg.h>
#include <string.h>
#include <tuple>

namespace fx {
static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

namespace {
struct ScratchBuf { void* ptr = nullptr; size_t bytes = 0; };
std::mutex g_scratch_mu;
std::map<std::tuple<int, hipStream_t, int>, ScratchBuf> g_scratch_map;
}  // namespace

int stream_scratch(ScratchKind kind, hipStream_t st, size_t bytes, void** out) {
    int dev = 0;
    FX_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    ScratchBuf& b = g_scratch_map[std::make_tuple(dev, st, (int)kind)];
    if (b.bytes < bytes) {
        if (b.ptr) {
            FX_HIP(hipStreamSynchronize(st));          // kernels queued earlier on this stream may still use the old buffer
            (void)hipFree(b.ptr);
            b = ScratchBuf();
        }
        const size_t want = (bytes + 255) & ~(size_t)255;
        hipError_t e = hipMalloc(&b.ptr, want);
        if (e != hipSuccess) {
            b = ScratchBuf();
            set_error("scratch hipMalloc(%zu) failed: %s", want, hipGetErrorString(e));
            return e == hipErrorOutOfMemory ? FLEXLLM_ENOMEM : FLEXLLM_EHIP;
        }
        b.bytes = want;
    }
    *out = b.ptr;
    return FLEXLLM_OK;
}

void stream_scratch_release(hipStream_t st) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    for (auto it = g_scratch_map.begin(); it != g_scratch_map.end();) {
        if (std::get<0>(it->first) == dev && std::get<1>(it->first) == st) {
            if (it->second.ptr) (void)hipFree(it->second.ptr);
            it = g_scratch_map.erase(it);
        } else {
            ++it;
        }
    }
}

// SplitMix64 of (seed, index): the same sequence as flexllm_amd.synth.splitmix64 on the host.
__host__ __device__ inline uint64_t splitmix64(uint64_t seed, uint64_t idx) {
    uint64_t z = seed + (idx + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__host__ __device__ inline float u01(uint64_t z) { return (float)(z >> 40) * (1.0f / 16777216.0f); }

__global__ void fill_i8_kernel(int8_t* dst, size_t n, uint64_t seed, int lo, unsigned span) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = (int8_t)(lo + (int)((splitmix64(seed, i) >> 33) % span));
}
__global__ void fill_f32_kernel(float* dst, size_t n, uint64_t seed, float lo, float width) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = lo + width * u01(splitmix64(seed, i));
}
__global__ void fill_f16_kernel(__half* dst, size_t n, uint64_t seed, float lo, float width) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = __float2half_rn(lo + width * u01(splitmix64(seed, i)));
}
}  // namespace fx

using namespace fx;

extern "C" {

const char* flexllm_last_error(void) { return g_err; }
const char* flexllm_build_info(void) { return "libflexllm_hip 0.1 (gfx950, HIP)"; }

int flexllm_rt_device_count(int* count) {
    FX_REQUIRE(count, "count is null");
    FX_HIP(hipGetDeviceCount(count));
    return FLEXLLM_OK;
}
int flexllm_rt_device_name(char* buf, int buflen) {
    FX_REQUIRE(buf && buflen > 0, "bad buffer");
    hipDeviceProp_t p;
    FX_HIP(hipGetDeviceProperties(&p, 0));
    snprintf(buf, buflen, "%s (%s, %d CUs)", p.name, p.gcnArchName, p.multiProcessorCount);
    return FLEXLLM_OK;
}
int flexllm_rt_malloc(void** dptr, size_t bytes) {
    FX_REQUIRE(dptr, "dptr is null");
    hipError_t e = hipMalloc(dptr, bytes ? bytes : 1);
    if (e == hipErrorOutOfMemory) { set_error("hipMalloc(%zu) out of memory", bytes); return FLEXLLM_ENOMEM; }
    FX_HIP(e);
    return FLEXLLM_OK;
}
int flexllm_rt_mem_info(size_t* free_bytes, size_t* total_bytes) {
    FX_REQUIRE(free_bytes && total_bytes, "mem_info: null pointer");
    FX_HIP(hipMemGetInfo(free_bytes, total_bytes));
    return FLEXLLM_OK;
}
int flexllm_rt_free(void* dptr) { FX_HIP(hipFree(dptr)); return FLEXLLM_OK; }
int flexllm_rt_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
    FX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    FX_HIP(hipStreamSynchronize(as_stream(stream)));
    return FLEXLLM_OK;
}
int flexllm_rt_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
    FX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    FX_HIP(hipStreamSynchronize(as_stream(stream)));
    return FLEXLLM_OK;
}
int flexllm_rt_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
    FX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return FLEXLLM_OK;
}
int flexllm_rt_memset(void* dst, int value, size_t bytes, void* stream) {
    FX_HIP(hipMemsetAsync(dst, value, bytes, as_stream(stream)));
    return FLEXLLM_OK;
}
int flexllm_rt_stream_create(void** stream) {
    FX_REQUIRE(stream, "stream is null");
    hipStream_t s;
    FX_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return FLEXLLM_OK;
}
int flexllm_rt_stream_destroy(void* stream) {
    FX_HIP(hipStreamSynchronize(as_stream(stream)));
    stream_scratch_release(as_stream(stream));         // the stand-alone entry points' scratch of this stream
    FX_HIP(hipStreamDestroy(as_stream(stream)));
    return FLEXLLM_OK;
}
int flexllm_rt_stream_sync(void* stream) { FX_HIP(hipStreamSynchronize(as_stream(stream))); return FLEXLLM_OK; }
int flexllm_rt_device_sync(void) { FX_HIP(hipDeviceSynchronize()); return FLEXLLM_OK; }
int flexllm_rt_event_create(void** event) {
    FX_REQUIRE(event, "event is null");
    hipEvent_t e;
    FX_HIP(hipEventCreate(&e));
    *event = e;
    return FLEXLLM_OK;
}
int flexllm_rt_event_destroy(void* event) { FX_HIP(hipEventDestroy((hipEvent_t)event)); return FLEXLLM_OK; }
int flexllm_rt_event_record(void* event, void* stream) {
    FX_HIP(hipEventRecord((hipEvent_t)event, as_stream(stream)));
    return FLEXLLM_OK;
}
int flexllm_rt_event_sync(void* event) { FX_HIP(hipEventSynchronize((hipEvent_t)event)); return FLEXLLM_OK; }
int flexllm_rt_event_elapsed_ms(void* start, void* stop, float* ms) {
    FX_REQUIRE(ms, "ms is null");
    FX_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return FLEXLLM_OK;
}

static int fill_grid(size_t n) {
    size_t b = (n + 255) / 256;
    return (int)(b < 1 ? 1 : b > 8192 ? 8192 : b);
}
int flexllm_rt_fill_i8(int8_t* dst, size_t n, uint64_t seed, int lo, int hi, void* stream) {
    FX_REQUIRE(dst && lo >= -128 && hi <= 127 && lo <= hi, "fill_i8: bad range [%d,%d]", lo, hi);
    if (n == 0) return FLEXLLM_OK;
    fill_i8_kernel<<<fill_grid(n), 256, 0, as_stream(stream)>>>(dst, n, seed, lo, (unsigned)(hi - lo + 1));
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}
int flexllm_rt_fill_uniform_f32(float* dst, size_t n, uint64_t seed, float lo, float hi, void* stream) {
    FX_REQUIRE(dst, "fill_f32: null");
    if (n == 0) return FLEXLLM_OK;
    fill_f32_kernel<<<fill_grid(n), 256, 0, as_stream(stream)>>>(dst, n, seed, lo, hi - lo);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}
int flexllm_rt_fill_uniform_f16(uint16_t* dst, size_t n, uint64_t seed, float lo, float hi, void* stream) {
    FX_REQUIRE(dst, "fill_f16: null");
    if (n == 0) return FLEXLLM_OK;
    fill_f16_kernel<<<fill_grid(n), 256, 0, as_stream(stream)>>>((__half*)dst, n, seed, lo, hi - lo);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // extern "C"

// Context, memory, stream, event and graph entry points of the C ABI.
#include "common.h"

#include <atomic>

namespace pet {

static std::atomic<bool> g_init{false};
static int g_device = -1;

char *err_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}

int set_error(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err_buf(), 512, fmt, ap);
    va_end(ap);
    return status;
}

bool initialised() { return g_init.load(); }

// Library-owned scratch for split-K contractions: partial tiles and one arrival
// counter per output tile (zero between launches). Allocated once in pet_hip_init (the reference's
// PerfEngine likewise owns its cuDNN workspace, src/Graph/perf_engine.cc:31-42).
// Launches that use it must not overlap on different streams.
static float *g_ws = nullptr;
static int *g_cnt = nullptr;
constexpr size_t kWsElems = (size_t)8 << 20; // 32 MiB of floats
constexpr int kNumCounters = 16384;

static std::atomic<int> g_deterministic{-1};

bool deterministic() {
    int v = g_deterministic.load();
    if (v < 0) {
        const char *e = getenv("PET_HIP_DETERMINISTIC");
        v = e && atoi(e) != 0;
        g_deterministic.store(v);
    }
    return v != 0;
}

void splitk_workspace(float **ws, size_t *ws_elems, int **counters, int *num_counters) {
    *ws = g_ws;
    *ws_elems = g_ws ? kWsElems : 0;
    *counters = g_cnt;
    *num_counters = g_cnt ? kNumCounters : 0;
}

__global__ void fill_kernel(float *dst, float v, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride)
        dst[i] = v;
}

// Counter-based generator (splitmix64 finaliser on seed + index): any element
// can be produced independently, so the fill is one flat kernel.
__global__ void rand_uniform_kernel(float *dst, size_t n, uint64_t seed, float lo,
                                    float scale) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint64_t z = seed + 0x9E3779B97F4A7C15ull * (uint64_t)(i + 1);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z = z ^ (z >> 31);
        float u = (float)(z >> 40) * (1.0f / 16777216.0f);
        dst[i] = lo + scale * u;
    }
}

} // namespace pet

using namespace pet;

static inline unsigned grid_for(size_t n, unsigned block) {
    size_t g = (n + block - 1) / block;
    if (g > 65536)
        g = 65536;
    if (g == 0)
        g = 1;
    return (unsigned)g;
}

extern "C" {

int pet_hip_init(int device) {
    int count = 0;
    PET_HIP_CHECK(hipGetDeviceCount(&count));
    if (device < 0 || device >= count)
        return set_error(PET_HIP_ERR_INVALID, "device %d out of range (%d devices)", device,
                         count);
    PET_HIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    PET_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(PET_HIP_ERR_UNSUPPORTED,
                         "this library is built for gfx950 only, device is %s",
                         prop.gcnArchName);
    if (!g_ws) {
        PET_HIP_CHECK(hipMalloc((void **)&g_ws, kWsElems * sizeof(float)));
        PET_HIP_CHECK(hipMalloc((void **)&g_cnt, kNumCounters * sizeof(int)));
        PET_HIP_CHECK(hipMemset(g_cnt, 0, kNumCounters * sizeof(int)));
        PET_HIP_CHECK(hipDeviceSynchronize());
    }
    g_device = device;
    g_init.store(true);
    err_buf()[0] = 0;
    return PET_HIP_OK;
}

int pet_hip_shutdown(void) {
    if (!g_init.load())
        return PET_HIP_OK;
    PET_HIP_CHECK(hipDeviceSynchronize());
    if (g_ws) {
        PET_HIP_CHECK(hipFree(g_ws));
        PET_HIP_CHECK(hipFree(g_cnt));
        g_ws = nullptr;
        g_cnt = nullptr;
    }
    g_init.store(false);
    return PET_HIP_OK;
}

const char *pet_hip_last_error(void) { return err_buf(); }

int pet_hip_set_deterministic(int on) {
    pet::g_deterministic.store(on != 0);
    return PET_HIP_OK;
}

int pet_hip_get_deterministic(int *on) {
    if (!on)
        return set_error(PET_HIP_ERR_INVALID, "null result pointer");
    *on = pet::deterministic() ? 1 : 0;
    return PET_HIP_OK;
}

int pet_hip_device_info(char *arch, size_t arch_len, int *num_cu) {
    PET_REQUIRE_INIT();
    hipDeviceProp_t prop;
    PET_HIP_CHECK(hipGetDeviceProperties(&prop, g_device));
    if (arch && arch_len) {
        strncpy(arch, prop.gcnArchName, arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    if (num_cu)
        *num_cu = prop.multiProcessorCount;
    return PET_HIP_OK;
}

int pet_hip_malloc(void **dptr, size_t bytes) {
    PET_REQUIRE_INIT();
    if (!dptr)
        return set_error(PET_HIP_ERR_INVALID, "null out pointer");
    PET_HIP_CHECK(hipMalloc(dptr, bytes ? bytes : 4));
    return PET_HIP_OK;
}

int pet_hip_free(void *dptr) {
    PET_REQUIRE_INIT();
    if (dptr)
        PET_HIP_CHECK(hipFree(dptr));
    return PET_HIP_OK;
}

int pet_hip_memcpy_h2d(void *dst, const void *src, size_t bytes, pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    PET_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(s)));
    PET_HIP_CHECK(hipStreamSynchronize(as_stream(s)));
    return PET_HIP_OK;
}

int pet_hip_memcpy_d2h(void *dst, const void *src, size_t bytes, pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    PET_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(s)));
    PET_HIP_CHECK(hipStreamSynchronize(as_stream(s)));
    return PET_HIP_OK;
}

int pet_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    PET_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(s)));
    return PET_HIP_OK;
}

int pet_hip_fill_f32(float *dst, float value, size_t n, pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    if (n == 0)
        return PET_HIP_OK;
    if (!dst)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    hipLaunchKernelGGL(fill_kernel, dim3(grid_for(n, 256)), dim3(256), 0, as_stream(s), dst,
                       value, n);
    return check_launch("fill_kernel");
}

int pet_hip_rand_uniform_f32(float *dst, size_t n, uint64_t seed, float lo, float hi,
                             pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    if (n == 0)
        return PET_HIP_OK;
    if (!dst)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    hipLaunchKernelGGL(rand_uniform_kernel, dim3(grid_for(n, 256)), dim3(256), 0, as_stream(s),
                       dst, n, seed, lo, hi - lo);
    return check_launch("rand_uniform_kernel");
}

int pet_hip_stream_create(pet_hip_stream_t *s) {
    PET_REQUIRE_INIT();
    hipStream_t st;
    PET_HIP_CHECK(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    *s = (pet_hip_stream_t)st;
    return PET_HIP_OK;
}

int pet_hip_stream_destroy(pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    if (s)
        PET_HIP_CHECK(hipStreamDestroy(as_stream(s)));
    return PET_HIP_OK;
}

int pet_hip_stream_sync(pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    PET_HIP_CHECK(hipStreamSynchronize(as_stream(s)));
    return PET_HIP_OK;
}

int pet_hip_event_create(pet_hip_event_t *e) {
    PET_REQUIRE_INIT();
    hipEvent_t ev;
    PET_HIP_CHECK(hipEventCreate(&ev));
    *e = (pet_hip_event_t)ev;
    return PET_HIP_OK;
}

int pet_hip_event_destroy(pet_hip_event_t e) {
    PET_REQUIRE_INIT();
    if (e)
        PET_HIP_CHECK(hipEventDestroy((hipEvent_t)e));
    return PET_HIP_OK;
}

int pet_hip_event_record(pet_hip_event_t e, pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    PET_HIP_CHECK(hipEventRecord((hipEvent_t)e, as_stream(s)));
    return PET_HIP_OK;
}

int pet_hip_event_sync(pet_hip_event_t e) {
    PET_REQUIRE_INIT();
    PET_HIP_CHECK(hipEventSynchronize((hipEvent_t)e));
    return PET_HIP_OK;
}

int pet_hip_event_elapsed_ms(float *ms, pet_hip_event_t start, pet_hip_event_t stop) {
    PET_REQUIRE_INIT();
    PET_HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return PET_HIP_OK;
}

int pet_hip_graph_begin_capture(pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    if (!s)
        return set_error(PET_HIP_ERR_INVALID, "capture needs an explicit stream");
    PET_HIP_CHECK(hipStreamBeginCapture(as_stream(s), hipStreamCaptureModeThreadLocal));
    return PET_HIP_OK;
}

int pet_hip_graph_end_capture(pet_hip_stream_t s, pet_hip_graph_t *g) {
    PET_REQUIRE_INIT();
    hipGraph_t graph = nullptr;
    PET_HIP_CHECK(hipStreamEndCapture(as_stream(s), &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess)
        return set_error(PET_HIP_ERR_RUNTIME, "hipGraphInstantiate failed: %s",
                         hipGetErrorString(e));
    *g = (pet_hip_graph_t)exec;
    return PET_HIP_OK;
}

int pet_hip_graph_launch(pet_hip_graph_t g, pet_hip_stream_t s) {
    PET_REQUIRE_INIT();
    PET_HIP_CHECK(hipGraphLaunch((hipGraphExec_t)g, as_stream(s)));
    return PET_HIP_OK;
}

int pet_hip_graph_destroy(pet_hip_graph_t g) {
    PET_REQUIRE_INIT();
    if (g)
        PET_HIP_CHECK(hipGraphExecDestroy((hipGraphExec_t)g));
    return PET_HIP_OK;
}

int pet_hip_conv_out_dim(int i, int k, int p, int s, int d) {
    if (s <= 0)
        return -1;
    return (i - (k - s) * d + p * 2) / s;
}

} // extern "C"

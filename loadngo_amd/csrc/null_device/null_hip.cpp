// The null device (see hip/hip_runtime_api.h beside this file): host memory for device memory, launches
// recorded instead of run. Also stands in for lng_static.hip, whose fixed device array is a plain host
// array here. Test infrastructure for the host library; never part of liblng_hip.so.
#include <hip/hip_runtime_api.h>

#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "../lng_static.h"

struct lng_null_stream { int unused; };
struct lng_null_event { int unused; };
struct lng_null_module { int unused; };
struct lng_null_function { std::string name; };

namespace {
struct Launch {
    std::string name;
    unsigned grid[3];
    unsigned block[3];
    std::vector<char> args;
};
std::mutex g_mu;
std::vector<Launch> g_launches;
std::map<const char *, size_t> g_allocations; // base -> size, device and pinned alike
std::map<std::string, lng_null_function> g_functions; // kernel names handed out as functions (nodes never move)
size_t g_fail_after = 0;

hipError_t allocate(void **ptr, size_t size, bool may_fail) {
    if (!ptr) return hipErrorInvalidValue;
    std::lock_guard<std::mutex> lock(g_mu);
    if (may_fail && g_fail_after && --g_fail_after == 0) {
        *ptr = nullptr;
        return hipErrorOutOfMemory;
    }
    void *p = malloc(size ? size : 1);
    if (!p) return hipErrorOutOfMemory;
    memset(p, 0xA5, size ? size : 1); // contents unspecified: make it show
    g_allocations[(const char *)p] = size;
    *ptr = p;
    return hipSuccess;
}

hipError_t release(void *ptr) {
    if (!ptr) return hipSuccess;
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_allocations.find((const char *)ptr);
    if (it == g_allocations.end()) return hipErrorInvalidValue;
    g_allocations.erase(it);
    free(ptr);
    return hipSuccess;
}
} // namespace

extern "C" {

const char *hipGetErrorString(hipError_t e) {
    switch (e) {
    case hipSuccess: return "no error";
    case hipErrorOutOfMemory: return "out of memory";
    case hipErrorInvalidDevice: return "invalid device";
    case hipErrorNotFound: return "not found";
    default: return "invalid value";
    }
}
hipError_t hipGetLastError(void) { return hipSuccess; }
hipError_t hipInit(unsigned) { return hipSuccess; }
hipError_t hipGetDeviceCount(int *count) {
    *count = 1;
    return hipSuccess;
}
hipError_t hipSetDevice(int device) { return device == 0 ? hipSuccess : hipErrorInvalidDevice; }
hipError_t hipGetDevice(int *device) {
    *device = 0;
    return hipSuccess;
}
hipError_t hipGetDeviceProperties(hipDeviceProp_t *prop, int) {
    memset(prop, 0, sizeof *prop);
    strcpy(prop->gcnArchName, "null-device");
    prop->multiProcessorCount = 256;
    return hipSuccess;
}
hipError_t hipDeviceSynchronize(void) { return hipSuccess; }

hipError_t hipMalloc(void **ptr, size_t size) { return allocate(ptr, size, true); }
hipError_t hipFree(void *ptr) { return release(ptr); }
hipError_t hipHostMalloc(void **ptr, size_t size, unsigned) { return allocate(ptr, size, false); }
hipError_t hipHostFree(void *ptr) { return release(ptr); }
hipError_t hipMemcpy(void *dst, const void *src, size_t size, hipMemcpyKind) {
    if (size) memcpy(dst, src, size);
    return hipSuccess;
}
hipError_t hipMemcpyAsync(void *dst, const void *src, size_t size, hipMemcpyKind kind, hipStream_t) { return hipMemcpy(dst, src, size, kind); }
hipError_t hipMemset(void *dst, int value, size_t size) {
    if (size) memset(dst, value, size);
    return hipSuccess;
}
hipError_t hipMemsetAsync(void *dst, int value, size_t size, hipStream_t) { return hipMemset(dst, value, size); }

hipError_t hipStreamCreateWithFlags(hipStream_t *stream, unsigned) {
    *stream = new lng_null_stream{0};
    return hipSuccess;
}
hipError_t hipStreamDestroy(hipStream_t stream) {
    delete stream;
    return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipEventCreate(hipEvent_t *event) {
    *event = new lng_null_event{0};
    return hipSuccess;
}
hipError_t hipEventDestroy(hipEvent_t event) {
    delete event;
    return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float *ms, hipEvent_t, hipEvent_t) {
    *ms = 0.0f;
    return hipSuccess;
}

hipError_t hipModuleLoad(hipModule_t *module, const char *) {
    *module = new lng_null_module{0};
    return hipSuccess;
}
hipError_t hipModuleLoadData(hipModule_t *module, const void *) {
    *module = new lng_null_module{0};
    return hipSuccess;
}
hipError_t hipModuleUnload(hipModule_t module) {
    delete module;
    return hipSuccess;
}
hipError_t hipModuleGetFunction(hipFunction_t *function, hipModule_t, const char *name) {
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_functions.find(name);
    if (it == g_functions.end()) it = g_functions.emplace(name, lng_null_function{name}).first;
    *function = &it->second;
    return hipSuccess;
}
hipError_t hipModuleLaunchKernel(hipFunction_t f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by, unsigned bz,
                                 unsigned, hipStream_t, void **, void **extra) {
    if (!f || !extra || extra[0] != HIP_LAUNCH_PARAM_BUFFER_POINTER || extra[2] != HIP_LAUNCH_PARAM_BUFFER_SIZE ||
        extra[4] != HIP_LAUNCH_PARAM_END) {
        return hipErrorInvalidValue;
    }
    // what the real runtime refuses: an empty grid or block, more than 1024 threads, a grid dimension past its limit
    if (!gx || !gy || !gz || !bx || !by || !bz || (uint64_t)bx * by * bz > 1024u || gx > 0x7fffffffu || gy > 65535u || gz > 65535u) {
        return hipErrorInvalidValue;
    }
    Launch l;
    l.name = f->name;
    l.grid[0] = gx, l.grid[1] = gy, l.grid[2] = gz;
    l.block[0] = bx, l.block[1] = by, l.block[2] = bz;
    const size_t size = *(const size_t *)extra[3];
    l.args.assign((const char *)extra[1], (const char *)extra[1] + size);
    std::lock_guard<std::mutex> lock(g_mu);
    g_launches.push_back(std::move(l));
    return hipSuccess;
}

size_t lng_null_launch_count(void) {
    std::lock_guard<std::mutex> lock(g_mu);
    return g_launches.size();
}
int lng_null_launch(size_t i, const char **name, unsigned grid[3], unsigned block[3], const void **args, size_t *args_size) {
    std::lock_guard<std::mutex> lock(g_mu);
    if (i >= g_launches.size()) return -1;
    const Launch &l = g_launches[i];
    if (name) *name = l.name.c_str();
    for (int d = 0; d < 3; ++d) {
        if (grid) grid[d] = l.grid[d];
        if (block) block[d] = l.block[d];
    }
    if (args) *args = l.args.data();
    if (args_size) *args_size = l.args.size();
    return 0;
}
void lng_null_clear(void) {
    std::lock_guard<std::mutex> lock(g_mu);
    g_launches.clear();
}
size_t lng_null_bytes_from(const void *p) {
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_allocations.upper_bound((const char *)p);
    if (it == g_allocations.begin()) return 0;
    --it;
    const char *base = it->first;
    if ((const char *)p >= base + it->second) return 0;
    return it->second - (size_t)((const char *)p - base);
}
size_t lng_null_live_allocations(void) {
    std::lock_guard<std::mutex> lock(g_mu);
    return g_allocations.size();
}
void lng_null_fail_malloc_after(size_t n) {
    std::lock_guard<std::mutex> lock(g_mu);
    g_fail_after = n;
}

// ---- the stand-in for lng_static.hip: the fixed scratch array is host memory ---------------------------
static unsigned char g_static_scratch[LNG_STATIC_SCRATCH_BYTES];
int lng_static_scratch_setup(int device) { return device == 0 ? (int)hipSuccess : (int)hipErrorInvalidDevice; }
void *lng_static_scratch(int device) { return device == 0 ? g_static_scratch : nullptr; }

} // extern "C"

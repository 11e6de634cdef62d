// The library's fixed device scratch: split-K partials for the entry point that allocates nothing
// (lng_hip_attention_grouped_static). The array lives in the image of this file's code object, one copy
// per GPU at that GPU's own address; it is zero when the code object is loaded and afterwards keeps
// whatever the last call left.
//
// In host code the array's NAME is a host-side stand-in, not a device address. The only thing host code
// may do with it is ask the runtime where the current device's copy is: lng_static_scratch_setup does
// that once per device, keeps the address, and every other host use goes through that address.
#include <hip/hip_runtime.h>

#include "lng_static.h"

static __device__ __align__(256) unsigned char scratch[LNG_STATIC_SCRATCH_BYTES];

namespace {
void *g_scratch_ptr[LNG_STATIC_MAX_DEVICES]; // device address of `scratch` on each device, NULL until set up
}

// With `device` current: finds this device's copy of the array. Idempotent. Returns a hipError_t as int.
extern "C" int lng_static_scratch_setup(int device) {
    if (device < 0 || device >= LNG_STATIC_MAX_DEVICES) return (int)hipErrorInvalidDevice;
    if (g_scratch_ptr[device]) return (int)hipSuccess;
    int current = -1;
    hipError_t e = hipGetDevice(&current);
    if (e != hipSuccess) return (int)e;
    if (current != device) return (int)hipErrorInvalidDevice;
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[device] = ptr;
    return (int)hipSuccess;
}

// The address lng_static_scratch_setup found for `device`, or NULL.
extern "C" void *lng_static_scratch(int device) {
    if (device < 0 || device >= LNG_STATIC_MAX_DEVICES) return nullptr;
    return g_scratch_ptr[device];
}

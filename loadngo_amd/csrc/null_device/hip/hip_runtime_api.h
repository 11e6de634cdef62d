/*
 * The null device: a stand-in for the few HIP runtime entry points the host library (lng_hip.cpp) uses, so
 * that the library's host logic - shape and slice refusals, ownership, the decode planner and its work
 * tables, scratch sizing, batch and completion handling - builds and runs on a machine without a GPU, under
 * AddressSanitizer and UndefinedBehaviorSanitizer (`python -m loadngo_amd.build --null-device`).
 *
 * Device memory is host memory (malloc), copies and fills happen at once, events hold nothing, and a kernel
 * launch is RECORDED, not run: its name, grid, block and a copy of its argument block go to a log the tests
 * read (lng_null_*). Only the host build defines LNG_NULL_DEVICE and puts this directory ahead of ROCm's on
 * the include path; the product never sees this file. Nothing here computes attention: there is no CPU
 * fallback.
 */
#ifndef LNG_NULL_HIP_RUNTIME_API_H
#define LNG_NULL_HIP_RUNTIME_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum hipError_t {
    hipSuccess = 0,
    hipErrorInvalidValue = 1,
    hipErrorOutOfMemory = 2,
    hipErrorInvalidDevice = 101,
    hipErrorNotFound = 500
} hipError_t;

typedef struct lng_null_stream *hipStream_t;
typedef struct lng_null_event *hipEvent_t;
typedef struct lng_null_module *hipModule_t;
typedef struct lng_null_function *hipFunction_t;

typedef enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2 } hipMemcpyKind;

typedef struct hipDeviceProp_t {
    char gcnArchName[256];
    int multiProcessorCount;
} hipDeviceProp_t;

#define hipStreamNonBlocking 1u
#define hipHostMallocDefault 0u
#define HIP_LAUNCH_PARAM_BUFFER_POINTER ((void *)0x01)
#define HIP_LAUNCH_PARAM_BUFFER_SIZE ((void *)0x02)
#define HIP_LAUNCH_PARAM_END ((void *)0x03)

const char *hipGetErrorString(hipError_t e);
hipError_t hipGetLastError(void);
hipError_t hipInit(unsigned flags);
hipError_t hipGetDeviceCount(int *count);
hipError_t hipSetDevice(int device);
hipError_t hipGetDevice(int *device);
hipError_t hipGetDeviceProperties(hipDeviceProp_t *prop, int device);
hipError_t hipDeviceSynchronize(void);

hipError_t hipMalloc(void **ptr, size_t size);
hipError_t hipFree(void *ptr);
hipError_t hipHostMalloc(void **ptr, size_t size, unsigned flags);
hipError_t hipHostFree(void *ptr);
hipError_t hipMemcpy(void *dst, const void *src, size_t size, hipMemcpyKind kind);
hipError_t hipMemcpyAsync(void *dst, const void *src, size_t size, hipMemcpyKind kind, hipStream_t stream);
hipError_t hipMemset(void *dst, int value, size_t size);
hipError_t hipMemsetAsync(void *dst, int value, size_t size, hipStream_t stream);

hipError_t hipStreamCreateWithFlags(hipStream_t *stream, unsigned flags);
hipError_t hipStreamDestroy(hipStream_t stream);
hipError_t hipStreamSynchronize(hipStream_t stream);
hipError_t hipEventCreate(hipEvent_t *event);
hipError_t hipEventDestroy(hipEvent_t event);
hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream);
hipError_t hipEventSynchronize(hipEvent_t event);
hipError_t hipEventElapsedTime(float *ms, hipEvent_t start, hipEvent_t stop);

hipError_t hipModuleLoad(hipModule_t *module, const char *path);
hipError_t hipModuleLoadData(hipModule_t *module, const void *image);
hipError_t hipModuleUnload(hipModule_t module);
hipError_t hipModuleGetFunction(hipFunction_t *function, hipModule_t module, const char *name);
hipError_t hipModuleLaunchKernel(hipFunction_t f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by, unsigned bz,
                                 unsigned shared_bytes, hipStream_t stream, void **params, void **extra);

/* ---- what the tests read ------------------------------------------------------------------------------ */

/* Launches recorded since the last lng_null_clear, oldest first. */
size_t lng_null_launch_count(void);
/* Launch i: the kernel's name, its grid and block, and its argument block (valid until lng_null_clear). */
int lng_null_launch(size_t i, const char **name, unsigned grid[3], unsigned block[3], const void **args, size_t *args_size);
void lng_null_clear(void);
/* Bytes from `p` to the end of the live hipMalloc allocation that holds it; 0 when none does. */
size_t lng_null_bytes_from(const void *p);
/* Live hipMalloc / hipHostMalloc allocations (leak checks). */
size_t lng_null_live_allocations(void);
/* The next `n`-th hipMalloc from now fails once (n = 1: the very next); 0 switches it off. */
void lng_null_fail_malloc_after(size_t n);

#ifdef __cplusplus
}
#endif
#endif /* LNG_NULL_HIP_RUNTIME_API_H */

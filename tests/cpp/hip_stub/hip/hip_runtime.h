// Host-only stand-in for the few HIP runtime calls the host side of the library
// (fbgemm_amd/csrc/c_api.cpp) makes, so that its plan / cache / scratch lifetime
// code can run on the CPU under the address and undefined-behaviour sanitizers
// (tests/test_host_sanitizers.py). "Device" memory is malloc'ed host memory, so a
// use after free, a double free, a leak or an overrun of it is the sanitizers' to
// find. Kernel launches do nothing (tests/cpp/hip_stub/hip_stub.cpp). Test
// infrastructure: nothing of the product is built against this file.
#pragma once
#include <stddef.h>
#include <stdint.h>

#define __device__
#define __host__
#define __global__
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&(x))

typedef int hipError_t;
enum : int { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2, hipErrorStreamCaptureUnsupported = 900 };
typedef struct hipStubStream* hipStream_t;
typedef struct hipStubEvent* hipEvent_t;
enum hipMemcpyKind { hipMemcpyHostToHost = 0, hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
enum hipStreamCaptureStatus { hipStreamCaptureStatusNone = 0, hipStreamCaptureStatusActive = 1 };
enum : unsigned { hipStreamNonBlocking = 1, hipEventDisableTiming = 2, hipEventDefault = 0 };

hipError_t hipMalloc(void** p, size_t bytes);
hipError_t hipFree(void* p);
hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind);
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind kind, hipStream_t stream);
hipError_t hipMemsetAsync(void* dst, int value, size_t bytes, hipStream_t stream);
hipError_t hipStreamSynchronize(hipStream_t stream);
hipError_t hipDeviceSynchronize(void);
hipError_t hipGetDevice(int* dev);
hipError_t hipGetLastError(void);
const char* hipGetErrorString(hipError_t e);
hipError_t hipStreamIsCapturing(hipStream_t stream, hipStreamCaptureStatus* status);
hipError_t hipStreamCreateWithFlags(hipStream_t* stream, unsigned flags);
hipError_t hipStreamDestroy(hipStream_t stream);
hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t event, unsigned flags);
hipError_t hipEventCreateWithFlags(hipEvent_t* event, unsigned flags);
hipError_t hipEventDestroy(hipEvent_t event);
hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream);
hipError_t hipEventSynchronize(hipEvent_t event);
hipError_t hipEventElapsedTime(float* ms, hipEvent_t start, hipEvent_t stop);
hipError_t hipGetSymbolAddressStub(void** p, const void* symbol);
#define hipGetSymbolAddress(p, sym) hipGetSymbolAddressStub((p), (const void*)(sym))

// ---- what the tests steer -------------------------------------------------------
// Streams for which hipStreamIsCapturing says "active" (a stand-in for hipStreamBeginCapture).
void hip_stub_set_capturing(hipStream_t stream, bool on);
// The n-th hipMalloc from now on fails (0 = the next one; negative = none fails).
void hip_stub_fail_malloc_after(long n);
// Device allocations alive, allocations and launches made so far.
long hip_stub_live_allocations(void);
long hip_stub_total_allocations(void);
long hip_stub_launches(void);
long hip_stub_wide4_launches(void); // launches of the lean kernel's four-waves-per-SIMD instance
// what hipEventElapsedTime reports from now on: `general_ms` for a measurement of a forward whose last lean launch was
// the general-purpose kernel, `wide4_ms` for one of the four-wave instance
void hip_stub_set_elapsed_ms(float general_ms, float wide4_ms);
// A stream handle that stands for a caller's stream (never dereferenced).
hipStream_t hip_stub_stream(int id);

// The few HIP names the library's host-side headers mention, for building host-only logic (tests/host_cpp/*_check.cpp) with a
// plain C++ compiler and its sanitizers.  Nothing here runs on a device and nothing of the library's device code is built with it.
#pragma once
#include <stddef.h>
typedef struct fake_hip_stream* hipStream_t;
typedef struct fake_hip_event* hipEvent_t;
typedef int hipError_t;
enum { hipSuccess = 0 };
static inline const char* hipGetErrorString(hipError_t) { return "host build"; }
static inline hipError_t hipGetLastError() { return hipSuccess; }

// Host stand-ins for the few device-side names the kernel template uses, so that the exact text
// the library hands to hipRTC can also be compiled for the CPU and run under AddressSanitizer.
// The template has no LDS and no barriers, so lanes can run one after another.
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstring>

#define __device__
#define __global__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)

struct sa_cpu_dim3 { unsigned int x, y, z; };
static sa_cpu_dim3 blockIdx, threadIdx, gridDim, blockDim;

struct float2 { float x, y; };
static inline int __popc(unsigned int v) { return __builtin_popcount(v); }

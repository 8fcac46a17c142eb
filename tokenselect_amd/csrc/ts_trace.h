// Development instrumentation of the fused selection kernel, compiled in by -DTS_TRACE
// only (the product build never includes this file): every workgroup notes the device
// clock at the marks of its phases, and ts_debug_trace() copies the notes to the host.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

__device__ uint64_t g_trace[4096 * 24];
extern "C" int ts_debug_trace(void* out, size_t bytes) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_trace), bytes);
}
#define TS_MARK(i)                                                                              \
  do {                                                                                          \
    if (threadIdx.x == 0)                                                                       \
      g_trace[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 24 + (i)] = wall_clock64();       \
  } while (0)

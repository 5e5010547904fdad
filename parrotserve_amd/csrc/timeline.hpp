// Profiling build only (python -m parrotserve_amd.build --timeline): force-included in front of prefix_mfma.hip, it
// turns the PH_TL(i) marks of the fused decode kernel into per-wave timestamps (constant 100 MHz clock) in a
// device array that ph_timeline_read copies out.  The product library is built without this file and its marks
// compile to nothing.
#pragma once
#include <hip/hip_runtime.h>

constexpr int kTimelineWaves = 4096, kTimelineMarks = 12;
__device__ unsigned long long ph_timeline_buf[kTimelineWaves * kTimelineMarks];
// the same marks in shader-clock ticks: a mark pair then also gives the clock rate the compute unit held between them
__device__ unsigned long long ph_timeline_clk[kTimelineWaves * kTimelineMarks];

#define PH_TL(i)                                                                                        \
  do {                                                                                                  \
    const unsigned tl_wg = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;              \
    const unsigned tl_wave = tl_wg * (blockDim.x >> 6) + (threadIdx.x >> 6);                            \
    if ((threadIdx.x & 63) == 0 && tl_wave < kTimelineWaves) {                                          \
      ph_timeline_buf[tl_wave * kTimelineMarks + (i)] = wall_clock64();                                 \
      ph_timeline_clk[tl_wave * kTimelineMarks + (i)] = clock64();                                      \
    }                                                                                                   \
  } while (0)

// host: copy the marks out ([waves][marks] uint64 ticks of 10 ns, 0 = mark not reached) / clear them
extern "C" int ph_timeline_read(void* host, size_t bytes) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(ph_timeline_buf), bytes);
}
extern "C" int ph_timeline_read_clocks(void* host, size_t bytes) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(ph_timeline_clk), bytes);
}
extern "C" int ph_timeline_clear(void) {
  void* p = nullptr;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(ph_timeline_buf)) != hipSuccess) return -1;
  return (int)hipMemset(p, 0, sizeof(ph_timeline_buf));
}

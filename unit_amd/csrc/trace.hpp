// Wave timelines of the kernels, for the build that `make trace` produces (libunit_amd_trace.so, -DUNIT_TRACE_BUILD).
// In the product build every UNIT_TRACE(...) expands to nothing.
//
// An instrumented kernel takes one more argument, a device buffer of kTraceWords 64-bit words per wave, and lane 0
// of every wave writes its stamps there before it ends: words 0 .. 7 are s_memrealtime stamps (a 100 MHz counter
// common to the whole device) at the points the kernel names, the others are the kernel's own counts (shader
// clock ticks from s_memtime, hardware ids).  python -m unit_amd.timeline reads the buffer and prints percentiles.
#pragma once
#ifdef UNIT_TRACE_BUILD
namespace unit {
constexpr int kTraceWords = 16;
constexpr int kTraceWaves = 1 << 15;
unsigned long long *trace_buffer();  // host side: the buffer given to unit_trace_set(), or null

struct WaveTrace {
  unsigned long long w[kTraceWords];
  __device__ __forceinline__ WaveTrace() {
#pragma unroll
    for (int i = 0; i < kTraceWords; ++i) w[i] = 0;
  }
  __device__ __forceinline__ void mark(int k) { w[k] = __builtin_amdgcn_s_memrealtime(); }
  __device__ __forceinline__ static unsigned long long ticks() { return __builtin_amdgcn_s_memtime(); }
  // wave_index: a dense index over the grid's waves
  __device__ __forceinline__ void flush(unsigned long long *buf, int wave_index) {
    if (buf == nullptr || wave_index >= kTraceWaves || (threadIdx.x & 63) != 0) return;
    unsigned hw, xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    w[14] = hw;
    w[15] = xcc;
#pragma unroll
    for (int i = 0; i < kTraceWords; ++i) buf[(size_t)wave_index * kTraceWords + i] = w[i];
  }
};
}  // namespace unit
#define UNIT_TRACE(...) __VA_ARGS__
#else
#define UNIT_TRACE(...)
#endif

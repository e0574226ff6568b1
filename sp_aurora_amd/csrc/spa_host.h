// Host-side helpers shared by the launchers: per-device facts read once, the
// dynamic-LDS attribute of a kernel set once per device, and the kernel-variant
// overrides of spa_tune().  Nothing here allocates device memory.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>

constexpr int SPA_MAX_DEVICES = 64;

// Variant overrides for experiments and tests (set through spa_tune, never read from the
// environment); 0 = the library's own choice.
enum {
  SPA_KNOB_FWD_GROUPS = 0,    // 1 | 2 wave groups per forward workgroup
  SPA_KNOB_FWD_SHARE = 1,     // 1: private K/V buffers per group, 2: 256-row workgroups sharing them
  SPA_KNOB_BWD_DQ_WAVES = 2,  // 4 | 8 waves per workgroup of the backward's dq kernel
  SPA_KNOB_BWD_DKDV_FORM = 3, // 1: compiler-scheduled MFMAs in the D = 128 dk/dv kernel (test twin)
  SPA_KNOB_FWD32_SPLIT = 4,   // 1: never the 32-row fp32 forward whose waves share the key tiles, 2: whenever D <= 64
  SPA_KNOB_FEW_ROWS = 5,     // 1: a key-split forward of up to 4 query rows stays on the MFMA kernels
  SPA_KNOB_COUNT = 6
};
extern std::atomic<int> g_spa_knob[SPA_KNOB_COUNT];
static inline int spa_knob(int k) { return g_spa_knob[k].load(std::memory_order_relaxed); }

// The current device, or -1.
static inline int spa_current_device() {
  int dev = -1;
  return hipGetDevice(&dev) == hipSuccess ? dev : -1;
}

// Compute units of the current device (256 when the query fails), cached per device.
static inline int spa_device_cus() {
  static std::atomic<int> cache[SPA_MAX_DEVICES];
  const int dev = spa_current_device();
  if (dev >= 0 && dev < SPA_MAX_DEVICES) {
    const int c = cache[dev].load(std::memory_order_relaxed);
    if (c > 0) return c;
  }
  int n = 0;
  if (dev < 0 || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
  if (dev >= 0 && dev < SPA_MAX_DEVICES) cache[dev].store(n, std::memory_order_relaxed);
  return n;
}

// hipFuncAttributeMaxDynamicSharedMemorySize of `kernel`, set the first time the kernel is
// launched on a device instead of at every launch.  One instantiation (and one flag word)
// per kernel: the kernel is a template VALUE parameter.
template <auto kernel>
hipError_t spa_allow_dynamic_lds(int smem) {
  static std::atomic<unsigned long long> ready{0};  // bit d: done on device d
  const int dev = spa_current_device();
  if (dev >= 0 && dev < SPA_MAX_DEVICES && ((ready.load(std::memory_order_acquire) >> dev) & 1ull)) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  if (e == hipSuccess && dev >= 0 && dev < SPA_MAX_DEVICES) ready.fetch_or(1ull << dev, std::memory_order_release);
  return e;
}

// Shared helpers of the HIP backend: error capture, stream cast, launch checks.
#ifndef CAVS_CSRC_COMMON_H_
#define CAVS_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "cavs_hip.h"

namespace cavs {

int set_error(int code, const char *fmt, ...);

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kWave = 64;
int num_cus();  // compute units of the current device (256 on MI355X)
// Device address of the built-in split-K scratch on the current device (looked up once per
// device; defined next to the array in gemm_kernels.hip).  `out` may be null.
int static_scratch_setup(float **out);

// Timing probe of the calling thread (cavs_profile_arm): while armed, the first kernel an
// entry point launches records `start` when it begins and every kernel records `stop` when
// it ends, so the pair brackets exactly the device time of the entry point's kernels.
struct LaunchProbe {
  hipEvent_t start = nullptr, stop = nullptr;
  bool armed = false, started = false;
};
LaunchProbe &launch_probe();

// Every kernel of this library is launched through here.
template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t st, Args &&...args) {
  LaunchProbe &p = launch_probe();
  if (p.armed) {
    hipEvent_t s = p.started ? nullptr : p.start;
    p.started = true;
    hipExtLaunchKernelGGL(kernel, grid, block, (unsigned)lds, st, s, p.stop, 0, static_cast<KArgs>(args)...);
  } else {
    hipLaunchKernelGGL(kernel, grid, block, (unsigned)lds, st, static_cast<KArgs>(args)...);
  }
}

}  // namespace cavs

#define CAVS_HIP_TRY(expr)                                                          \
  do {                                                                              \
    hipError_t _e = (expr);                                                         \
    if (_e != hipSuccess)                                                           \
      return cavs::set_error(CAVS_EHIP, "%s failed: %s (%s:%d)", #expr,             \
                             hipGetErrorString(_e), __FILE__, __LINE__);            \
  } while (0)

#define CAVS_REQUIRE(cond, ...)                                   \
  do {                                                            \
    if (!(cond)) return cavs::set_error(CAVS_EINVAL, __VA_ARGS__); \
  } while (0)

// after a kernel launch
#define CAVS_LAUNCH_CHECK() CAVS_HIP_TRY(hipGetLastError())

#endif

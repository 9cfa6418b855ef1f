// Generic fused elementwise op: compiles the source emitted by the fusion pass with
// the HIP runtime compiler for gfx950 and launches it over a 1-D grid.  The source
// dialect (extern "C" __global__, blockIdx/threadIdx, atomicAdd, expf/tanhf) is the
// one the reference's generator emits and is valid HIP as is.
#include <hip/hiprtc.h>

#include <string>
#include <vector>

#include "common.h"

namespace cavs {

struct FusedKernel {
  hipModule_t module = nullptr;
  hipFunction_t fn = nullptr;
  std::string name;
};

constexpr int kFusedBlock = 256;

}  // namespace cavs

using namespace cavs;

extern "C" {

int cavs_fused_compile(const char *kernel_name, const char *source, void **handle) {
  CAVS_REQUIRE(kernel_name && source && handle, "cavs_fused_compile: null argument");
  *handle = nullptr;
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, (std::string(kernel_name) + ".hip").c_str(), 0,
                                       nullptr, nullptr);
  if (r != HIPRTC_SUCCESS)
    return set_error(CAVS_EHIP, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
  // FMA contraction off: the reference builds fused kernels with --fmad=false
  const char *opts[] = {"--offload-arch=gfx950", "-O3", "-ffp-contract=off"};
  r = hiprtcCompileProgram(prog, 3, opts);
  if (r != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    return set_error(CAVS_EINVAL, "hiprtc compile of %s failed: %.380s", kernel_name, log.c_str());
  }
  size_t code_size = 0;
  hiprtcGetCodeSize(prog, &code_size);
  std::vector<char> code(code_size);
  hiprtcGetCode(prog, code.data());
  hiprtcDestroyProgram(&prog);
  FusedKernel *k = new FusedKernel;
  k->name = kernel_name;
  hipError_t e = hipModuleLoadData(&k->module, code.data());
  if (e == hipSuccess) e = hipModuleGetFunction(&k->fn, k->module, kernel_name);
  if (e != hipSuccess) {
    if (k->module) (void)hipModuleUnload(k->module);
    delete k;
    return set_error(CAVS_EHIP, "loading fused kernel %s: %s", kernel_name, hipGetErrorString(e));
  }
  *handle = k;
  return CAVS_OK;
}

int cavs_fused_launch(void *handle, float *const *outs, int nouts, const float *const *ins, int nins,
                      const int *out_counts, const int *in_counts, int n_elements, void *stream) {
  CAVS_REQUIRE(handle, "cavs_fused_launch: null handle");
  CAVS_REQUIRE(nouts >= 0 && nins >= 0 && nouts + nins > 0 && n_elements >= 0,
               "cavs_fused_launch: bad counts (nouts=%d nins=%d n=%d)", nouts, nins, n_elements);
  if (n_elements == 0) return CAVS_OK;
  FusedKernel *k = static_cast<FusedKernel *>(handle);
  // argument order: outputs, inputs, output counts, input counts, n_elements
  std::vector<void *> ptrs(nouts + nins);
  std::vector<int> counts(nouts + nins);
  std::vector<void *> args;
  for (int i = 0; i < nouts; i++) {
    CAVS_REQUIRE(outs[i] && out_counts[i] > 0, "cavs_fused_launch: bad output %d", i);
    ptrs[i] = outs[i];
    counts[i] = out_counts[i];
  }
  for (int i = 0; i < nins; i++) {
    CAVS_REQUIRE(ins[i] && in_counts[i] > 0, "cavs_fused_launch: bad input %d", i);
    ptrs[nouts + i] = const_cast<float *>(ins[i]);
    counts[nouts + i] = in_counts[i];
  }
  for (auto &p : ptrs) args.push_back(&p);
  for (auto &c : counts) args.push_back(&c);
  args.push_back(&n_elements);
  unsigned grid = (unsigned)((n_elements + kFusedBlock - 1) / kFusedBlock);
  LaunchProbe &p = launch_probe();
  if (p.armed) {
    hipEvent_t s = p.started ? nullptr : p.start;
    p.started = true;
    CAVS_HIP_TRY(hipExtModuleLaunchKernel(k->fn, grid * kFusedBlock, 1, 1, kFusedBlock, 1, 1, 0, as_stream(stream),
                                          args.data(), nullptr, s, p.stop, 0));
  } else {
    CAVS_HIP_TRY(hipModuleLaunchKernel(k->fn, grid, 1, 1, kFusedBlock, 1, 1, 0, as_stream(stream),
                                       args.data(), nullptr));
  }
  return CAVS_OK;
}

int cavs_fused_release(void *handle) {
  if (!handle) return CAVS_OK;
  FusedKernel *k = static_cast<FusedKernel *>(handle);
  hipError_t e = hipModuleUnload(k->module);
  delete k;
  CAVS_HIP_TRY(e);
  return CAVS_OK;
}

}  // extern "C"

// Generic fused elementwise op: compiles the source emitted by the fusion pass with
// the HIP runtime compiler for gfx950 and launches it over a 1-D grid.  The source
// dialect (extern "C" __global__, blockIdx/threadIdx, atomicAdd, expf/tanhf) is the
// one the reference's generator emits and is valid HIP as is.
#include <hip/hiprtc.h>

#include <map>
#include <mutex>
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

// A vertex function's generated round kernels: one module, its kernels by a fixed order of names.
constexpr int kCellKernels = 8;
const char *const kCellKernelNames[kCellKernels] = {"cell_fwd",       "cell_leaves", "cell_bwd",       "cell_bwd_rows",
                                                    "cell_pack",      "cell_bias",   "cell_bwd_gates", "cell_bwd_pool"};
struct CellModule {
  hipModule_t module = nullptr;
  hipFunction_t fn[kCellKernels] = {};
  int users = 0;
  std::string source;
};
// Compiled modules by source: sessions that declare the same vertex function, at the same time or
// one after the other, share one (a compile is about a second).  Guarded by a mutex; a module
// without users stays loaded until more than kCellModulesKept are.
constexpr size_t kCellModulesKept = 32;
std::mutex &cell_mutex() {
  static std::mutex m;
  return m;
}
std::map<std::string, CellModule *> &cell_modules() {
  static std::map<std::string, CellModule *> m;
  return m;
}

// compiles `source` for gfx950 into `code`; the log of a failed compile goes into the error text
int rtc_compile(const char *what, const char *source, std::vector<char> *code) {
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, (std::string(what) + ".hip").c_str(), 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return set_error(CAVS_EHIP, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
  // FMA contraction off: the reference builds fused kernels with --fmad=false; packed fp32 math is
  // disabled on this target by policy
  const char *opts[] = {"--offload-arch=gfx950", "-O3", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  r = hiprtcCompileProgram(prog, 7, opts);
  if (r != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    return set_error(CAVS_EINVAL, "hiprtc compile of %s failed: %.380s", what, log.c_str());
  }
  size_t code_size = 0;
  hiprtcGetCodeSize(prog, &code_size);
  code->resize(code_size);
  hiprtcGetCode(prog, code->data());
  hiprtcDestroyProgram(&prog);
  return CAVS_OK;
}

}  // namespace cavs

using namespace cavs;

extern "C" {

int cavs_fused_compile(const char *kernel_name, const char *source, void **handle) {
  CAVS_REQUIRE(kernel_name && source && handle, "cavs_fused_compile: null argument");
  *handle = nullptr;
  std::vector<char> code;
  if (int rc = rtc_compile(kernel_name, source, &code)) return rc;
  FusedKernel *k = new FusedKernel;
  k->name = kernel_name;
  hipError_t e = hipModuleLoadData(&k->module, code.data());
  if (e == hipSuccess) e = hipModuleGetFunction(&k->fn, k->module, kernel_name);
  if (e != hipSuccess) {
    if (k->module) (void)hipModuleUnload(k->module);
    delete k;
    (void)hipGetLastError();  // reported here; not left behind for the next caller of the runtime
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

int cavs_cell_compile(const char *source, void **handle) {
  CAVS_REQUIRE(source && handle, "cavs_cell_compile: null argument");
  *handle = nullptr;
  std::lock_guard<std::mutex> lock(cell_mutex());
  auto it = cell_modules().find(source);
  if (it != cell_modules().end()) {
    it->second->users++;
    *handle = it->second;
    return CAVS_OK;
  }
  std::vector<char> code;
  if (int rc = rtc_compile("cell", source, &code)) return rc;
  CellModule *m = new CellModule;
  hipError_t e = hipModuleLoadData(&m->module, code.data());
  for (int i = 0; i < kCellKernels && e == hipSuccess; i++) e = hipModuleGetFunction(&m->fn[i], m->module, kCellKernelNames[i]);
  if (e != hipSuccess) {
    if (m->module) (void)hipModuleUnload(m->module);
    delete m;
    (void)hipGetLastError();  // reported here; not left behind for the next caller of the runtime
    return set_error(CAVS_EHIP, "loading the generated round kernels: %s", hipGetErrorString(e));
  }
  m->users = 1;
  m->source = source;
  cell_modules()[m->source] = m;
  *handle = m;
  return CAVS_OK;
}

int cavs_cell_launch(void *handle, int kernel, unsigned grid_x, unsigned grid_y, unsigned grid_z, unsigned block, const void *args,
                     size_t args_bytes, void *stream) {
  CAVS_REQUIRE(handle && args, "cavs_cell_launch: null argument");
  CAVS_REQUIRE(kernel >= 0 && kernel < kCellKernels, "cavs_cell_launch: no kernel %d", kernel);
  CAVS_REQUIRE(block >= 64 && block <= 256 && block % 64 == 0 && args_bytes > 0 && args_bytes <= 4096,
               "cavs_cell_launch: bad launch shape (block=%u, %zu argument bytes)", block, args_bytes);
  if (grid_x == 0 || grid_y == 0 || grid_z == 0) return CAVS_OK;
  CellModule *m = static_cast<CellModule *>(handle);
  // the kernels take one struct by value: its bytes are the argument buffer
  size_t bytes = args_bytes;
  void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void *>(args), HIP_LAUNCH_PARAM_BUFFER_SIZE, &bytes, HIP_LAUNCH_PARAM_END};
  LaunchProbe &p = launch_probe();
  if (p.armed) {
    hipEvent_t s = p.started ? nullptr : p.start;
    p.started = true;
    CAVS_HIP_TRY(hipExtModuleLaunchKernel(m->fn[kernel], grid_x * block, grid_y, grid_z, block, 1, 1, 0, as_stream(stream), nullptr, config,
                                          s, p.stop, 0));
  } else {
    CAVS_HIP_TRY(hipModuleLaunchKernel(m->fn[kernel], grid_x, grid_y, grid_z, block, 1, 1, 0, as_stream(stream), nullptr, config));
  }
  return CAVS_OK;
}

int cavs_cell_release(void *handle) {
  if (!handle) return CAVS_OK;
  CellModule *m = static_cast<CellModule *>(handle);
  std::lock_guard<std::mutex> lock(cell_mutex());
  if (--m->users > 0 || cell_modules().size() <= kCellModulesKept) return CAVS_OK;
  cell_modules().erase(m->source);
  hipError_t e = hipModuleUnload(m->module);
  delete m;
  CAVS_HIP_TRY(e);
  return CAVS_OK;
}

}  // extern "C"

// The entry point that allocates nothing, and the static device scratch array
// it works in.  Compiled by hipcc as host + device code (the array has to be a
// registered device symbol); everything else in the library is host-only C++
// or a raw code object.
#include "internal.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>

namespace {

// One copy per GPU, held from the moment the library's code object is loaded
// on that GPU until the process ends.  The compiler gives a static device
// variable that host code refers to external linkage in the code object, which
// is how the runtime finds it by name; attributes that pin its linkage
// (`used`) keep it local there, and the lookup then aborts inside the runtime.
constexpr size_t kScratchBytes = HCAMD_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// `scratch` in host code is a stand-in for the symbol, not an address: the
// address of each GPU's copy comes from hipGetSymbolAddress and is kept here.
constexpr int kMaxDevices = 64;
void *g_scratchOn[kMaxDevices] = {nullptr};

} // namespace

extern "C" {

int hcamdInternalScratchSetup(int device, char *err, size_t errLen) noexcept {
  if (device < 0 || device >= kMaxDevices) {
    std::snprintf(err, errLen, "device index %d (scratch is kept for indices below %d)", device,
                  kMaxDevices);
    return 1;
  }
  if (g_scratchOn[device])
    return 0;
  void *ptr = nullptr;
  const hipError_t rc = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (rc != hipSuccess || !ptr) {
    std::snprintf(err, errLen, "'hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))' failed with '%s'",
                  hipGetErrorName(rc));
    return 1;
  }
  g_scratchOn[device] = ptr;
  return 0;
}

int hcamdLaunchMapReduceColsNoAlloc(OlQueue q, int kind, const HcamdMapInstr *prog, size_t nInstr,
                                    const HcamdMapInstr *post, size_t nPost,
                                    const void *const *inputs, const int *inputTypes,
                                    const size_t *inputLd, size_t nInputs, void *out, int outType,
                                    size_t rows, size_t cols) noexcept {
  const char *who = "hcamdLaunchMapReduceColsNoAlloc";
  const int device = hcamdInternalQueueDeviceIndex(q);
  if (device < 0)
    return 1;
  void *ptr = device < kMaxDevices ? g_scratchOn[device] : nullptr;
  if (!ptr) {
    hcamdInternalReport(q, "%s: no scratch array on device %d (its address is looked up when the "
                           "device is created, for device indices below %d)", who, device, kMaxDevices);
    return 1;
  }
  if (!hcamdInternalColsKernelsReady(q)) {
    hcamdInternalReport(q, "%s: kernels of device %d were not resolved at creation", who, device);
    return 1;
  }
  const size_t need = hcamdMapReduceColsWorkspace(rows, cols);
  if (need > kScratchBytes) {
    hcamdInternalReport(q, "%s: a %zu x %zu window needs %zu bytes of scratch, the limit is %zu",
                        who, rows, cols, need, kScratchBytes);
    return 1;
  }
  // Every band cell the second launch reads is written by the first, so the
  // previous call's contents need no clearing.
  return hcamdLaunchMapReduceCols(q, kind, prog, nInstr, post, nPost, inputs, inputTypes, inputLd,
                                  nInputs, out, outType, rows, cols, ptr, kScratchBytes);
}

} // extern "C"

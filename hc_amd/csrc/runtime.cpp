// libhc_amd_runtime.so: the offload ABI (ol*), the launch half of the Python
// runtime ABI (hcgpu*) and the typed launchers (hcamd*) for one MI355X, written
// directly on the HIP module API: hipModuleLoadData, hipModuleGetFunction,
// hipModuleLaunchKernel, one stream per queue, hipMalloc.  The signatures and
// the reference interfaces they replace are documented in
// include/hc_amd_runtime.h; the measurement entry points are declared in
// include/hc_amd_bench.h.
#include "hc_amd_runtime.h"
#include "hc_amd_bench.h"
#include "internal.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

namespace {

// ---------------------------------------------------------------------------
// Call tracing (Loader.cpp:41-149, PyRuntime.cpp:12-34): "<fn> enter" /
// "<fn> exit" on stdout, flushed, so that a trace interleaves correctly with
// Python's own output.
// ---------------------------------------------------------------------------
bool g_traceLoader = false;
bool g_tracePy = false;

struct Scope {
  Scope(const char *fn, bool on) : name(fn), enabled(on) {
    if (enabled) {
      std::fprintf(stdout, "%s enter\n", name);
      std::fflush(stdout);
    }
  }
  Scope(const char *fn, bool on, const char *fmt, ...) : name(fn), enabled(on) {
    if (!enabled)
      return;
    std::fprintf(stdout, "%s ", name);
    va_list ap;
    va_start(ap, fmt);
    std::vfprintf(stdout, fmt, ap);
    va_end(ap);
    std::fprintf(stdout, "\n");
    std::fflush(stdout);
  }
  Scope(const Scope &) = delete;
  ~Scope() {
    if (enabled) {
      std::fprintf(stdout, "%s exit\n", name);
      std::fflush(stdout);
    }
  }
  const char *name;
  bool enabled;
};
#define OL_TRACE() Scope scope_(__func__, g_traceLoader)
#define PY_TRACE() Scope scope_(__func__, g_tracePy)

std::vector<std::string> g_searchPaths;

// ---------------------------------------------------------------------------
// Handles
// ---------------------------------------------------------------------------
struct Device {
  OlErrorCallback callback = nullptr;
  void *ctx = nullptr;
  int index = 0;
  int computeUnits = 0; // filled in on first use
  bool colsKernelsReady = false; // the column-reduction kernels were resolved at creation
  // one byte per row for the row programs that take two launches (which rows the
  // first one left to the second); allocated on first use, grown when needed
  void *rowMarks = nullptr;
  size_t rowMarksBytes = 0;
  // built-in modules and kernels, loaded on first use
  std::unordered_map<std::string, hipModule_t> modules;
  std::unordered_map<std::string, struct Kernel *> kernels;
  std::mutex cacheLock; // guards the two maps

  void report(const char *fmt, ...) {
    if (!callback)
      return;
    char buf[256] = {0};
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(buf, sizeof(buf) - 1, fmt, ap);
    va_end(ap);
    callback(ctx, OL_SEVERITY_ERROR, buf);
  }
  // 0 on success; otherwise reports "'<expr>' failed with '<hipErrorName>'"
  int check(const char *expr, hipError_t err) {
    if (err == hipSuccess)
      return 0;
    const char *name = hipGetErrorName(err);
    report("'%s' failed with '%s'\n", expr, name ? name : "<unknown>");
    return 1;
  }
  int makeCurrent() { return check("hipSetDevice(index)", hipSetDevice(index)); }
  ~Device();
};
#define HIP_CHECK(dev, expr) (dev)->check(#expr, (expr))

struct Module {
  Device *device = nullptr;
  hipModule_t module = nullptr;
};

struct Kernel {
  Device *device = nullptr;
  hipFunction_t function = nullptr;
  std::string name;
};

struct Queue {
  Device *device = nullptr;
  hipStream_t stream = nullptr;
};

struct Event {
  Device *device = nullptr;
  hipStream_t stream = nullptr;
  hipEvent_t event = nullptr;
};

Device::~Device() {
  for (auto &kv : kernels)
    delete kv.second;
  for (auto &kv : modules)
    if (kv.second)
      (void)hipModuleUnload(kv.second);
}

// ---------------------------------------------------------------------------
// Built-in code objects, linked in by blobs.S.
// ---------------------------------------------------------------------------
#define HCAMD_BLOB(n)                                                          \
  extern "C" const unsigned char hcamd_blob_##n##_begin[];                     \
  extern "C" const unsigned char hcamd_blob_##n##_end[];
HCAMD_BLOB(copy)
HCAMD_BLOB(elementwise)
HCAMD_BLOB(map)
HCAMD_BLOB(imap)
HCAMD_BLOB(fmap)
HCAMD_BLOB(distance)
HCAMD_BLOB(gather)
HCAMD_BLOB(softmax)
HCAMD_BLOB(quantize)
HCAMD_BLOB(gemm)
#undef HCAMD_BLOB

struct Blob {
  const char *name;
  const unsigned char *begin;
  const unsigned char *end;
};
#define HCAMD_BLOB(n) {#n, hcamd_blob_##n##_begin, hcamd_blob_##n##_end}
const Blob kBlobs[] = {HCAMD_BLOB(copy), HCAMD_BLOB(elementwise),
                       HCAMD_BLOB(map), HCAMD_BLOB(imap), HCAMD_BLOB(fmap), HCAMD_BLOB(distance),
                       HCAMD_BLOB(gather), HCAMD_BLOB(softmax),
                       HCAMD_BLOB(quantize), HCAMD_BLOB(gemm)};
#undef HCAMD_BLOB
constexpr size_t kNumBlobs = sizeof(kBlobs) / sizeof(kBlobs[0]);

Kernel *builtinKernel(Device *dev, const char *moduleName,
                      const char *kernelName) {
  std::string key = std::string(moduleName) + ":" + kernelName;
  std::lock_guard<std::mutex> guard(dev->cacheLock);
  auto it = dev->kernels.find(key);
  if (it != dev->kernels.end())
    return it->second;
  if (dev->makeCurrent())
    return nullptr;
  hipModule_t mod = nullptr;
  auto mit = dev->modules.find(moduleName);
  if (mit != dev->modules.end()) {
    mod = mit->second;
  } else {
    const Blob *blob = nullptr;
    for (const Blob &b : kBlobs)
      if (std::strcmp(b.name, moduleName) == 0)
        blob = &b;
    if (!blob) {
      dev->report("Unknown built-in module '%s'", moduleName);
      return nullptr;
    }
    if (HIP_CHECK(dev, hipModuleLoadData(&mod, blob->begin)))
      return nullptr;
    dev->modules.emplace(moduleName, mod);
  }
  hipFunction_t fn = nullptr;
  if (dev->check(kernelName, hipModuleGetFunction(&fn, mod, kernelName)))
    return nullptr;
  auto *k = new Kernel{dev, fn, kernelName};
  dev->kernels.emplace(std::move(key), k);
  return k;
}

// ---------------------------------------------------------------------------
// Launch helper shared by olLaunchKernel and the typed launchers.
// ---------------------------------------------------------------------------
thread_local const char *t_lastKernel = "";

int launch(Queue *q, Kernel *k, const size_t grid[3], const size_t block[3],
           void **args, size_t sharedMem) {
  Device *dev = q->device;
  for (int i = 0; i < 3; ++i) {
    if (grid[i] == 0 || block[i] == 0) {
      dev->report("Empty launch dimension for '%s'", k->name.c_str());
      return 1;
    }
  }
  if (grid[0] > 0x7fffffffull || grid[1] > 65535 || grid[2] > 65535 ||
      block[0] * block[1] * block[2] > 1024) {
    dev->report("Launch geometry out of range for '%s': grid %zu,%zu,%zu "
                "block %zu,%zu,%zu",
                k->name.c_str(), grid[0], grid[1], grid[2], block[0], block[1],
                block[2]);
    return 1;
  }
  t_lastKernel = k->name.c_str();
  return HIP_CHECK(
      dev, hipModuleLaunchKernel(k->function, (unsigned)grid[0],
                                 (unsigned)grid[1], (unsigned)grid[2],
                                 (unsigned)block[0], (unsigned)block[1],
                                 (unsigned)block[2], (unsigned)sharedMem,
                                 q->stream, args, nullptr));
}

int launch1d(Queue *q, const char *module, const char *name, size_t groups,
             size_t threads, void **args) {
  Kernel *k = builtinKernel(q->device, module, name);
  if (!k)
    return 1;
  const size_t grid[3] = {groups, 1, 1}, block[3] = {threads, 1, 1};
  return launch(q, k, grid, block, args, 0);
}

int computeUnitsOf(Device *dev) {
  if (dev->computeUnits == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount,
                              dev->index) != hipSuccess || n <= 0)
      n = 256;
    dev->computeUnits = n;
  }
  return dev->computeUnits;
}

inline bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}
inline size_t ceilDiv(size_t a, size_t b) { return (a + b - 1) / b; }

uint32_t upPow2(uint32_t x) {
  x--;
  x |= x >> 1;
  x |= x >> 2;
  x |= x >> 4;
  x |= x >> 8;
  x |= x >> 16;
  return x + 1;
}

// kernel-variant overrides (0 = choose by shape)
std::unordered_map<std::string, int> &variants() {
  static std::unordered_map<std::string, int> v{
      {"add", 0},     {"fma", 0},  {"softmax", 0},
      {"quantize", 0}, {"gemm", 0}, {"copy", 0}, {"map", 0},
      {"gather", 0}, {"gather_fuse", 0}, {"rows", 0}, {"stream", 0}, {"cols", 0}, {"norm", 0}};
  return v;
}
std::mutex g_variantLock; // guards variants()
// Per-thread overrides: a thread that launches with a variant of its own (a
// tuned kernel object) neither disturbs nor sees what other threads selected.
thread_local std::unordered_map<std::string, int> t_variants;

int variantOf(const char *family) {
  if (!t_variants.empty()) {
    auto it = t_variants.find(family);
    if (it != t_variants.end())
      return it->second;
  }
  std::lock_guard<std::mutex> guard(g_variantLock);
  auto &v = variants();
  auto it = v.find(family);
  return it == v.end() ? 0 : it->second;
}

// ---------------------------------------------------------------------------
// Process-wide device and queue of the hcgpu* entry points
// (GpuRuntime.cpp:23-24).
// ---------------------------------------------------------------------------
OlDevice g_device = nullptr;
OlQueue g_queue = nullptr;

void stderrCallback(void *, OlSeverity sev, const char *desc) {
  static const char *const kinds[] = {"error", "warning", "message"};
  const char *kind = (sev >= 0 && sev <= 2) ? kinds[sev] : "error";
  std::fprintf(stderr, "Offload %s: %s\n", kind, desc);
  std::fflush(stderr);
}

[[noreturn]] void fatal(const char *desc) {
  stderrCallback(nullptr, OL_SEVERITY_ERROR, desc);
  std::abort();
}

// 0 ok, otherwise the name of the step that failed
const char *ensureDefaultQueue(const char *deviceDesc) {
  static std::mutex lock;
  std::lock_guard<std::mutex> guard(lock);
  if (g_device)
    return nullptr;
  OlDevice dev = olCreateDevice(deviceDesc, &stderrCallback, nullptr);
  if (!dev)
    return "olCreateDevice failed";
  OlQueue q = olCreateQueue(dev);
  if (!q) {
    olReleaseDevice(dev);
    return "olCreateSyncQueue failed";
  }
  g_device = dev;
  g_queue = q;
  return nullptr;
}

} // namespace

// ===========================================================================
// 1. Offload ABI
// ===========================================================================
extern "C" {

void setGPULoaderSearchPaths(const char *paths[], size_t count) noexcept {
  g_searchPaths.clear();
  for (size_t i = 0; i < count; ++i)
    g_searchPaths.emplace_back(paths[i] ? paths[i] : "");
}

void enableFuncTracing(int val) noexcept { g_traceLoader = val != 0; }

OlDevice olCreateDevice(const char *desc, OlErrorCallback errCallback,
                        void *ctx) noexcept {
  OL_TRACE();
  auto fail = [&](const std::string &msg) -> OlDevice {
    if (errCallback)
      errCallback(ctx, OL_SEVERITY_ERROR, msg.c_str());
    return nullptr;
  };
  if (!desc)
    return fail("Invalid device desc: <null>");
  const std::string d(desc);
  const size_t sep = d.find(':');
  if (sep == std::string::npos)
    return fail("Invalid device desc: " + d);
  const std::string runtime = d.substr(0, sep);
  if (runtime != "hip")
    return fail("Runtime not found: " + runtime);
  const std::string id = d.substr(sep + 1);
  if (id.empty() || id.find_first_not_of("0123456789") != std::string::npos ||
      id.size() > 6)
    return fail("Invalid device id");

  auto dev = std::make_unique<Device>();
  dev->callback = errCallback;
  dev->ctx = ctx;
  dev->index = std::atoi(id.c_str());
  if (dev->makeCurrent())
    return nullptr;
  // Set-up for the entry point that allocates nothing: this GPU's address of the
  // static scratch array, and the kernels it launches.  A failure here only
  // makes that entry point refuse; every other one works without either.
  // (Its failure is not this call's: the device is created, and the entry point
  // says why it cannot run when it is called.)
  char why[200] = {0};
  if (!hcamdInternalScratchSetup(dev->index, why, sizeof(why))) {
    dev->colsKernelsReady = true;
    // every kernel a column reduction can launch, whatever the "cols" variant
    for (const char *name : {"hcamd_map_reduce_cols_n1u4", "hcamd_map_reduce_cols_n2u2",
                             "hcamd_map_reduce_cols_n4u1", "hcamd_cols_sum_f32",
                             "hcamd_cols_sumsq_f32", "hcamd_cols_sum_f32_w4u8",
                             "hcamd_cols_sumsq_f32_w4u8", "hcamd_cols_fold_f32"})
      if (!builtinKernel(dev.get(), "map", name))
        dev->colsKernelsReady = false;
  }
  return dev.release();
}

void olReleaseDevice(OlDevice dev) noexcept {
  OL_TRACE();
  auto *device = static_cast<Device *>(dev);
  if (device && device->rowMarks)
    (void)hipFree(device->rowMarks);
  delete device;
}

OlModule olCreateModule(OlDevice dev, const void *data,
                        size_t /*len*/) noexcept {
  OL_TRACE();
  auto *device = static_cast<Device *>(dev);
  if (!device)
    return nullptr;
  if (!data) {
    device->report("olCreateModule: null code object");
    return nullptr;
  }
  if (device->makeCurrent())
    return nullptr;
  hipModule_t mod = nullptr;
  if (HIP_CHECK(device, hipModuleLoadData(&mod, data)))
    return nullptr;
  return new Module{device, mod};
}

void olReleaseModule(OlModule mod) noexcept {
  OL_TRACE();
  auto *m = static_cast<Module *>(mod);
  if (!m)
    return;
  if (m->module)
    HIP_CHECK(m->device, hipModuleUnload(m->module));
  delete m;
}

OlKernel olGetKernel(OlModule mod, const char *name) noexcept {
  OL_TRACE();
  auto *m = static_cast<Module *>(mod);
  if (!m || !name)
    return nullptr;
  hipFunction_t fn = nullptr;
  if (HIP_CHECK(m->device, hipModuleGetFunction(&fn, m->module, name)))
    return nullptr;
  return new Kernel{m->device, fn, name};
}

void olReleaseKernel(OlKernel k) noexcept {
  OL_TRACE();
  delete static_cast<Kernel *>(k);
}

int olSuggestBlockSize(OlKernel /*k*/, const size_t *globalsSizes,
                       size_t *blockSizesRet, size_t nDims) noexcept {
  OL_TRACE();
  if (nDims < 1 || nDims > 3 || !globalsSizes || !blockSizesRet)
    return 1;
  size_t budget = 1024;
  for (size_t i = 0; i < nDims; ++i) {
    const size_t g = globalsSizes[i];
    if (g > 1) {
      // budget stays a power of two >= 1: l <= budget implies
      // upPow2(l) <= budget
      const size_t l = std::min(g, budget);
      blockSizesRet[i] = l;
      budget /= upPow2(static_cast<uint32_t>(l));
    } else {
      blockSizesRet[i] = 1;
    }
  }
  return 0;
}

OlQueue olCreateQueue(OlDevice dev) noexcept {
  OL_TRACE();
  auto *device = static_cast<Device *>(dev);
  if (!device || device->makeCurrent())
    return nullptr;
  hipStream_t stream = nullptr;
  if (HIP_CHECK(device, hipStreamCreate(&stream)))
    return nullptr;
  return new Queue{device, stream};
}

void olReleaseQueue(OlQueue q) noexcept {
  OL_TRACE();
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return;
  if (queue->stream)
    HIP_CHECK(queue->device, hipStreamDestroy(queue->stream));
  delete queue;
}

int olSyncQueue(OlQueue q) noexcept {
  OL_TRACE();
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  return HIP_CHECK(queue->device, hipStreamSynchronize(queue->stream));
}

void *olAllocDevice(OlQueue q, size_t size, size_t /*align*/) noexcept {
  OL_TRACE();
  auto *queue = static_cast<Queue *>(q);
  if (!queue || queue->device->makeCurrent())
    return nullptr;
  void *ptr = nullptr;
  if (HIP_CHECK(queue->device, hipMalloc(&ptr, size)))
    return nullptr;
  return ptr;
}

void olDeallocDevice(OlQueue q, void *data) noexcept {
  OL_TRACE();
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return;
  HIP_CHECK(queue->device, hipFree(data));
}

int olLaunchKernel(OlQueue q, OlKernel k, const size_t *gridSizes,
                   const size_t *blockSizes, size_t nDims, void **args,
                   size_t nArgs, size_t sharedMemSize) noexcept {
  Scope scope_(__func__, g_traceLoader,
               "grid: [%zu, %zu, %zu], blocks [%zu, %zu, %zu], nargs %zu, "
               "shMem %zu",
               nDims > 0 ? gridSizes[0] : 0, nDims > 1 ? gridSizes[1] : 0,
               nDims > 2 ? gridSizes[2] : 0, nDims > 0 ? blockSizes[0] : 0,
               nDims > 1 ? blockSizes[1] : 0, nDims > 2 ? blockSizes[2] : 0,
               nArgs, sharedMemSize);
  auto *queue = static_cast<Queue *>(q);
  auto *kernel = static_cast<Kernel *>(k);
  if (!queue || !kernel)
    return 1;
  if (nDims != 3) {
    queue->device->report("Invalid launch dims: %d", static_cast<int>(nDims));
    return 1;
  }
  return launch(queue, kernel, gridSizes, blockSizes, args, sharedMemSize);
}

// ===========================================================================
// 2. Python-runtime ABI, launch half
// ===========================================================================
void hcgpuEnableTraceFunctions(int val) noexcept { g_tracePy = val != 0; }

void *hcgpuGetKernel(void **handle, const char *deviceDesc, const void *data,
                     size_t dataSize, const char *kernelName) noexcept {
  PY_TRACE();
  if (handle && *handle)
    return *handle;
  if (const char *err = ensureDefaultQueue(deviceDesc))
    fatal(err);
  // The module is intentionally kept for the life of the process: the kernel
  // handle cached by the caller borrows from it (GpuRuntime.cpp:41-50).
  OlModule module = olCreateModule(g_device, data, dataSize);
  if (!module)
    fatal("olCreateModule failed");
  OlKernel kernel = olGetKernel(module, kernelName);
  if (!kernel)
    fatal("olGetKernel failed");
  if (handle)
    *handle = kernel;
  return kernel;
}

void hcgpuSuggestBlockSize(void *kernel, const size_t *globalSizes,
                           size_t *blockSizesRet, size_t nDim) noexcept {
  PY_TRACE();
  if (olSuggestBlockSize(kernel, globalSizes, blockSizesRet, nDim))
    fatal("olSuggestBlockSize failed");
}

void hcgpuLaunchKernel(void *kernel, const size_t *gridSizes,
                       const size_t *blockSizes, size_t nDim, void **args,
                       size_t nArgs, size_t sharedMemSize) noexcept {
  PY_TRACE();
  if (!g_queue)
    fatal("olLaunchKernel failed");
  if (olLaunchKernel(g_queue, kernel, gridSizes, blockSizes, nDim, args, nArgs,
                     sharedMemSize))
    fatal("olLaunchKernel failed");
  if (olSyncQueue(g_queue))
    fatal("olSyncQueue failed");
}

// ===========================================================================
// 3. Additions
// ===========================================================================
OlQueue hcamdGetDefaultQueue(const char *deviceDesc) noexcept {
  if (const char *err = ensureDefaultQueue(deviceDesc)) {
    stderrCallback(nullptr, OL_SEVERITY_ERROR, err);
    return nullptr;
  }
  return g_queue;
}

OlDevice hcamdGetDefaultDevice(const char *deviceDesc) noexcept {
  return hcamdGetDefaultQueue(deviceDesc) ? g_device : nullptr;
}

int hcamdInternalQueueDeviceIndex(OlQueue q) noexcept {
  return q ? static_cast<Queue *>(q)->device->index : -1;
}

void hcamdInternalReport(OlQueue q, const char *fmt, ...) noexcept {
  if (!q)
    return;
  char buf[256] = {0};
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof(buf) - 1, fmt, ap);
  va_end(ap);
  static_cast<Queue *>(q)->device->report("%s", buf);
}

int hcamdInternalColsKernelsReady(OlQueue q) noexcept {
  return q && static_cast<Queue *>(q)->device->colsKernelsReady ? 1 : 0;
}

OlDevice hcamdQueueDevice(OlQueue q) noexcept {
  return q ? static_cast<Queue *>(q)->device : nullptr;
}

size_t hcamdBuiltinModuleCount(void) noexcept { return kNumBlobs; }

int hcamdGetBuiltinModule(size_t index, const char **name, const void **data,
                          size_t *len) noexcept {
  if (index >= kNumBlobs)
    return 1;
  if (name)
    *name = kBlobs[index].name;
  if (data)
    *data = kBlobs[index].begin;
  if (len)
    *len = static_cast<size_t>(kBlobs[index].end - kBlobs[index].begin);
  return 0;
}

OlKernel hcamdGetBuiltinKernel(OlDevice dev, const char *moduleName,
                               const char *kernelName) noexcept {
  if (!dev || !moduleName || !kernelName)
    return nullptr;
  return builtinKernel(static_cast<Device *>(dev), moduleName, kernelName);
}

int hcamdMemcpy(OlQueue q, void *dst, const void *src, size_t bytes,
                int kind) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  static const hipMemcpyKind kinds[] = {hipMemcpyHostToDevice,
                                        hipMemcpyDeviceToHost,
                                        hipMemcpyDeviceToDevice};
  if (kind < 0 || kind > 2) {
    queue->device->report("Invalid copy kind: %d", kind);
    return 1;
  }
  if (bytes == 0)
    return 0;
  return HIP_CHECK(queue->device,
                   hipMemcpyAsync(dst, src, bytes, kinds[kind], queue->stream));
}

int hcamdFill32(OlQueue q, void *dst, uint32_t value, size_t count) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  if (count == 0)
    return 0;
  void *args[] = {&dst, &value, &count};
  return launch1d(queue, "copy", "hcamd_fill32", ceilDiv(count, 256), 256,
                  args);
}

HcamdEvent hcamdEventCreate(OlQueue q) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue || queue->device->makeCurrent())
    return nullptr;
  hipEvent_t ev = nullptr;
  if (HIP_CHECK(queue->device, hipEventCreate(&ev)))
    return nullptr;
  return new Event{queue->device, queue->stream, ev};
}

void hcamdEventDestroy(HcamdEvent e) noexcept {
  auto *ev = static_cast<Event *>(e);
  if (!ev)
    return;
  HIP_CHECK(ev->device, hipEventDestroy(ev->event));
  delete ev;
}

int hcamdEventRecord(HcamdEvent e) noexcept {
  auto *ev = static_cast<Event *>(e);
  if (!ev)
    return 1;
  return HIP_CHECK(ev->device, hipEventRecord(ev->event, ev->stream));
}

int hcamdEventSynchronize(HcamdEvent e) noexcept {
  auto *ev = static_cast<Event *>(e);
  if (!ev)
    return 1;
  return HIP_CHECK(ev->device, hipEventSynchronize(ev->event));
}

int hcamdEventElapsedMs(HcamdEvent start, HcamdEvent stop,
                        float *ms) noexcept {
  auto *a = static_cast<Event *>(start);
  auto *b = static_cast<Event *>(stop);
  if (!a || !b || !ms)
    return 1;
  return HIP_CHECK(a->device, hipEventElapsedTime(ms, a->event, b->event));
}

int hcamdDeviceInfo(OlDevice dev, int *computeUnits, int *clockKHz,
                    int *memClockKHz, int *memBusBits, size_t *totalMem,
                    char *archName, size_t archLen) noexcept {
  auto *device = static_cast<Device *>(dev);
  if (!device)
    return 1;
  hipDeviceProp_t prop;
  if (HIP_CHECK(device, hipGetDeviceProperties(&prop, device->index)))
    return 1;
  if (computeUnits)
    *computeUnits = prop.multiProcessorCount;
  if (clockKHz)
    *clockKHz = prop.clockRate;
  if (memClockKHz)
    *memClockKHz = prop.memoryClockRate;
  if (memBusBits)
    *memBusBits = prop.memoryBusWidth;
  if (totalMem)
    *totalMem = prop.totalGlobalMem;
  if (archName && archLen) {
    std::strncpy(archName, prop.gcnArchName, archLen - 1);
    archName[archLen - 1] = '\0';
  }
  return 0;
}

namespace {
// Variants 17..22, 26, 28, 29, 33 and 34 of "gemm" are measurement builds of the default
// kernel with one part of its loop taken out: what they leave in C is not the product
// (30..32 are further hand orders of variant 27 that only measurements select).
// They exist only in a library built with HCAMD_PROBES defined (`python -m
// hc_amd.build --probes`); any other build refuses to select them.
bool variantIsAbsentProbe(const char *family, int variant) {
#ifdef HCAMD_PROBES
  (void)family, (void)variant;
  return false;
#else
  return std::strcmp(family, "gemm") == 0 &&
         ((variant >= 17 && variant <= 22) || variant == 26 || (variant >= 28 && variant <= 34));
#endif
}
} // namespace

int hcamdProbesBuilt(void) noexcept {
#ifdef HCAMD_PROBES
  return 1;
#else
  return 0;
#endif
}

int hcamdSetVariant(const char *family, int variant) noexcept {
  if (!family || variantIsAbsentProbe(family, variant))
    return 1;
  std::lock_guard<std::mutex> guard(g_variantLock);
  auto &v = variants();
  auto it = v.find(family);
  if (it == v.end())
    return 1;
  it->second = variant;
  return 0;
}

int hcamdSetThreadVariant(const char *family, int variant) noexcept {
  if (!family || variantIsAbsentProbe(family, variant))
    return 1;
  {
    std::lock_guard<std::mutex> guard(g_variantLock);
    if (variants().find(family) == variants().end())
      return 1;
  }
  try {
    if (variant < 0)
      t_variants.erase(family);
    else
      t_variants[family] = variant;
  } catch (...) {
    return 1;
  }
  return 0;
}

const char *hcamdLastKernelName(void) noexcept { return t_lastKernel; }

// ---------------------------------------------------------------------------
// Typed launchers
// ---------------------------------------------------------------------------
int hcamdLaunchTranspose2D(OlQueue q, size_t elemSize, const void *src, size_t srcLd, void *dst,
                           size_t dstLd, size_t rows, size_t cols) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *name = elemSize == 1   ? "hcamd_transpose2d_b1"
                     : elemSize == 2 ? "hcamd_transpose2d_b2"
                     : elemSize == 4 ? "hcamd_transpose2d_b4"
                     : elemSize == 8 ? "hcamd_transpose2d_b8"
                                     : nullptr;
  if (!name) {
    dev->report("hcamdLaunchTranspose2D: unsupported element size %zu", elemSize);
    return 1;
  }
  if (rows == 0 || cols == 0)
    return 0;
  if (!src || !dst) {
    dev->report("hcamdLaunchTranspose2D: null pointer");
    return 1;
  }
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % elemSize) {
    dev->report("hcamdLaunchTranspose2D: pointer not aligned to the element size");
    return 1;
  }
  if ((rows > 1 && srcLd < cols) || (cols > 1 && dstLd < rows)) {
    dev->report("hcamdLaunchTranspose2D: leading dimension smaller than a row");
    return 1;
  }
  if (rows > 0xffffffffull || cols > 0xffffffffull || ceilDiv(rows, (size_t)64) > 65535) {
    dev->report("hcamdLaunchTranspose2D: window of %zu x %zu (at most 4,194,240 rows)", rows, cols);
    return 1;
  }
  Kernel *k = builtinKernel(dev, "copy", name);
  if (!k)
    return 1;
  uint32_t nRows = static_cast<uint32_t>(rows), nCols = static_cast<uint32_t>(cols);
  void *args[] = {&src, &srcLd, &dst, &dstLd, &nRows, &nCols};
  const size_t grid[3] = {ceilDiv(cols, (size_t)64), ceilDiv(rows, (size_t)64), 1};
  const size_t block[3] = {256, 1, 1};
  return launch(queue, k, grid, block, args, 0);
}

int hcamdLaunchCopy2D(OlQueue q, size_t elemSize, const void *src,
                      size_t srcRows, size_t srcCols, ptrdiff_t ss0,
                      ptrdiff_t ss1, void *dst, size_t dstRows, size_t dstCols,
                      ptrdiff_t ds0, ptrdiff_t ds1) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *suffix = nullptr;
  switch (elemSize) {
  case 1: suffix = "b1"; break;
  case 2: suffix = "b2"; break;
  case 4: suffix = "b4"; break;
  case 8: suffix = "b8"; break;
  case 16: suffix = "b16"; break;
  default:
    dev->report("hcamdLaunchCopy2D: unsupported element size %zu", elemSize);
    return 1;
  }
  size_t rows = std::min(srcRows, dstRows);
  size_t cols = std::min(srcCols, dstCols);
  if (rows == 0 || cols == 0)
    return 0;
  if (!src || !dst) {
    dev->report("hcamdLaunchCopy2D: null pointer");
    return 1;
  }
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) %
      elemSize) {
    dev->report("hcamdLaunchCopy2D: pointer not aligned to the element size");
    return 1;
  }
  // Window covers whole rows of both arrays and both are dense: one vector.
  const bool dense = ss1 == 1 && ds1 == 1 &&
                     (rows == 1 || (ss0 == (ptrdiff_t)cols &&
                                    ds0 == (ptrdiff_t)cols));
  const int variant = variantOf("copy");
  if (dense && aligned16(src) && aligned16(dst) && variant != 9) {
    static const char *const names[] = {
        "hcamd_copy_flat_v4_nt", "hcamd_copy_flat_v1",    "hcamd_copy_flat_v2",
        "hcamd_copy_flat_v4",    "hcamd_copy_flat_v8",    "hcamd_copy_flat_v1_nt",
        "hcamd_copy_flat_v2_nt", "hcamd_copy_flat_v4_nt", "hcamd_copy_flat_v8_nt"};
    static const int vpt[] = {4, 1, 2, 4, 8, 1, 2, 4, 8};
    const int v = (variant >= 0 && variant <= 8) ? variant : 0;
    size_t nbytes = rows * cols * elemSize;
    const size_t words = ceilDiv(nbytes, 16);
    void *args[] = {&src, &dst, &nbytes};
    return launch1d(queue, "copy", names[v], ceilDiv(words, 256 * (size_t)vpt[v]),
                    256, args);
  }
  // A window of rows that are contiguous inside: use the widest element both
  // arrays' rows are aligned for (an int32 window with even extents and strides
  // is an int64 window of half the width, and so on up to 16 bytes).
  if (ss1 == 1 && ds1 == 1 && variant != 9) {
    while (elemSize < 16 && cols % 2 == 0 &&
           (rows == 1 || (ss0 % 2 == 0 && ds0 % 2 == 0)) &&
           (reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) %
                   (2 * elemSize) == 0) {
      elemSize *= 2;
      cols /= 2;
      ss0 /= 2;
      ds0 /= 2;
    }
    suffix = elemSize == 1   ? "b1"
             : elemSize == 2 ? "b2"
             : elemSize == 4 ? "b4"
             : elemSize == 8 ? "b8"
                             : "b16";
  }
  // Rows that lie the same way against 16-byte boundaries in both arrays
  // (rows of whole 16-byte elements always do): aligned 16-byte pieces, with
  // ragged ends where the rows have them, non-temporal both ways (8192 x 8192
  // int32 of a stride-8200 array 92 -> 87 us, 8191 x 8191 at offset 1 160 -> 87 us;
  // variant 10 of "copy" keeps the element-wise kernel).
  // Rows that lie differently in the two arrays: the same pieces of the
  // destination, each read from wherever its 16 bytes are in the source.
  if (ss1 == 1 && ds1 == 1 && variant != 9 && variant != 10 && cols * elemSize >= 64) {
    const bool same =
        (reinterpret_cast<uintptr_t>(src) - reinterpret_cast<uintptr_t>(dst)) % 16 == 0 &&
        (rows == 1 || ((ss0 - ds0) * (ptrdiff_t)elemSize) % 16 == 0);
    Kernel *k = builtinKernel(dev, "copy", same ? "hcamd_copy2d_rows" : "hcamd_copy2d_rows_any");
    if (!k)
      return 1;
    size_t rowBytes = cols * elemSize;
    ptrdiff_t sb = ss0 * (ptrdiff_t)elemSize, db = ds0 * (ptrdiff_t)elemSize;
    const size_t pieces = rowBytes / 16 + 2; // whole pieces and the two ragged ends
    const size_t bx = pieces >= 256 ? 256 : 64, by = 256 / bx;
    for (size_t r0 = 0; r0 < rows; r0 += 65535 * by) {
      size_t nr = std::min(rows - r0, (size_t)65535 * by);
      const char *s = static_cast<const char *>(src) + (ptrdiff_t)r0 * sb;
      char *d = static_cast<char *>(dst) + (ptrdiff_t)r0 * db;
      void *args[] = {&s, &sb, &d, &db, &nr, &rowBytes};
      const size_t grid[3] = {ceilDiv(pieces, bx), ceilDiv(nr, by), 1};
      const size_t block[3] = {bx, by, 1};
      if (launch(queue, k, grid, block, args, 0))
        return 1;
    }
    return 0;
  }
  const std::string name = std::string("hcamd_copy2d_") + suffix;
  Kernel *k = builtinKernel(dev, "copy", name.c_str());
  if (!k)
    return 1;
  // rows go to grid.y (at most 65535 per launch): split tall windows
  const size_t bx = cols >= 256 ? 256 : 64, by = 256 / bx;
  for (size_t r0 = 0; r0 < rows; r0 += 65535 * by) {
    size_t nr = std::min(rows - r0, (size_t)65535 * by);
    const char *s = static_cast<const char *>(src) +
                    (ptrdiff_t)r0 * ss0 * (ptrdiff_t)elemSize;
    char *d = static_cast<char *>(dst) + (ptrdiff_t)r0 * ds0 * (ptrdiff_t)elemSize;
    void *args[] = {&s, &ss0, &ss1, &d, &ds0, &ds1, &nr, &cols};
    const size_t grid[3] = {ceilDiv(cols, bx), ceilDiv(nr, by), 1};
    const size_t block[3] = {bx, by, 1};
    if (launch(queue, k, grid, block, args, 0))
      return 1;
  }
  return 0;
}

namespace {
struct IdScatterArgs {
  void *out;
  int32_t out_type, out_rank, rank, per_item;
  int64_t out_shape[3], out_stride[3];
  int64_t idx_c[3], idx_g[3][3], idx_l[3][3];
  int64_t val_c, val_g[3], val_l[3];
};
} // namespace

int hcamdLaunchIdScatter(OlQueue q, void *out, int outType, size_t outRank,
                         const size_t *outShape, const ptrdiff_t *outStrides,
                         const HcamdAffineId *index, const HcamdAffineId *value, size_t rank,
                         const size_t *groupCount, const size_t *groupShape,
                         int perItem) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *who = "hcamdLaunchIdScatter";
  if (!out || !outShape || !outStrides || !index || !value || !groupCount || !groupShape) {
    dev->report("%s: null pointer", who);
    return 1;
  }
  if (rank < 1 || rank > 3 || outRank < 1 || outRank > 3) {
    dev->report("%s: ranks %zu / %zu (1..3)", who, rank, outRank);
    return 1;
  }
  IdScatterArgs a{};
  a.out = out;
  a.out_type = outType == HCAMD_I32 ? 0 : outType == HCAMD_I64 ? 1 : outType == HCAMD_F32 ? 2 : -1;
  if (a.out_type < 0) {
    dev->report("%s: unsupported output type %d", who, outType);
    return 1;
  }
  a.out_rank = (int32_t)outRank;
  a.rank = (int32_t)rank;
  a.per_item = perItem ? 1 : 0;
  size_t grid[3] = {1, 1, 1}, block[3] = {1, 1, 1}, threads = 1, groups = 1;
  for (size_t d = 0; d < rank; ++d) {
    // Python dimension d is hardware dimension rank - 1 - d
    grid[rank - 1 - d] = groupCount[d];
    block[rank - 1 - d] = groupShape[d];
    threads *= groupShape[d];
    groups *= groupCount[d];
  }
  if (groups == 0 || threads == 0)
    return 0;
  if (threads > 1024) {
    dev->report("%s: a group of %zu work-items (at most 1024 fit one workgroup)", who, threads);
    return 1;
  }
  if (grid[1] > 65535 || grid[2] > 65535 || grid[0] > 0x7fffffffull) {
    dev->report("%s: %zu x %zu x %zu groups (at most 65535 along every dimension but the last)", who,
                grid[2], grid[1], grid[0]);
    return 1;
  }
  for (size_t d = 0; d < outRank; ++d) {
    if (outShape[d] == 0)
      return 0;
    a.out_shape[d] = (int64_t)outShape[d];
    a.out_stride[d] = (int64_t)outStrides[d];
    a.idx_c[d] = index[d].c;
    for (int k = 0; k < 3; ++k) {
      a.idx_g[d][k] = index[d].g[k];
      a.idx_l[d][k] = index[d].l[k];
    }
  }
  a.val_c = value->c;
  for (int k = 0; k < 3; ++k) {
    a.val_g[k] = value->g[k];
    a.val_l[k] = value->l[k];
  }
  Kernel *k = builtinKernel(dev, "copy", "hcamd_id_scatter");
  if (!k)
    return 1;
  void *args[] = {&a};
  return launch(queue, k, grid, block, args, 0);
}

int hcamdLaunchStream(OlQueue q, int nReads, int writeMode, const void *const *inputs,
                      void *out, size_t bytes) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *name = nullptr;
  if (writeMode == HCAMD_STREAM_NONE && nReads == 1)
    name = "hcamd_stream_r1w0";
  else if (writeMode == HCAMD_STREAM_HALF && nReads == 1)
    name = "hcamd_stream_r1w1h";
  else if (writeMode == HCAMD_STREAM_FULL && nReads >= 0 && nReads <= 3) {
    static const char *const full[] = {"hcamd_stream_r0w1", "hcamd_stream_r1w1",
                                       "hcamd_stream_r2w1", "hcamd_stream_r3w1"};
    name = full[nReads];
  }
  if (!name) {
    dev->report("hcamdLaunchStream: no kernel for %d read stream(s) and write mode %d", nReads,
                writeMode);
    return 1;
  }
  if (bytes == 0)
    return 0;
  if (bytes % 16384 != 0 || bytes / 16384 > 0x7fffffffull) {
    dev->report("hcamdLaunchStream: %zu bytes (a multiple of 16 KiB, below 2^45)", bytes);
    return 1;
  }
  const void *in[3] = {nullptr, nullptr, nullptr};
  for (int i = 0; i < nReads; ++i) {
    if (!inputs || !inputs[i] || !aligned16(inputs[i])) {
      dev->report("hcamdLaunchStream: null or unaligned input %d", i);
      return 1;
    }
    in[i] = inputs[i];
  }
  if (!out || !aligned16(out)) {
    dev->report("hcamdLaunchStream: null or unaligned output");
    return 1;
  }
  void *args[] = {&in[0], &in[1], &in[2], &out};
  // 256-lane workgroups of one word a lane, paced as the fp16 fma kernel is
  // (four waves per SIMD and 6, 0 or 12 pauses before the store: "stream"
  // variants 2, 3, 4) or not paced at all (5).  By shape (variant 0) only three
  // reads against one write take the paced form: measured 85.8 -> 80.0 us at
  // 128 MiB a stream; every other mix is slower that way.  Variant 1: the
  // 512-lane form for every mix.
  static const char *const paced[] = {"_w4_d6", "_w4_d0", "_w4_d12", "_w8"};
  int variant = variantOf("stream");
  if (variant == 0 && nReads == 3)
    variant = 2;
  if (variant >= 2 && variant <= 5 && nReads > 0 && writeMode != HCAMD_STREAM_NONE) {
    char full[64];
    snprintf(full, sizeof full, "%s%s", name, paced[variant - 2]);
    return launch1d(queue, "copy", full, bytes / 4096, 256, args);
  }
  return launch1d(queue, "copy", name, bytes / 16384, 512, args);
}

int hcamdLaunchCopy2DTiled(OlQueue q, size_t elemSize, const void *src,
                           void *dst, size_t rows, size_t cols, ptrdiff_t ss0,
                           ptrdiff_t ds0, size_t blockX, size_t blockY,
                           size_t unroll) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *suffix = nullptr;
  switch (elemSize) {
  case 1: suffix = "b1"; break;
  case 2: suffix = "b2"; break;
  case 4: suffix = "b4"; break;
  case 8: suffix = "b8"; break;
  case 16: suffix = "b16"; break;
  default:
    dev->report("hcamdLaunchCopy2DTiled: unsupported element size %zu",
                elemSize);
    return 1;
  }
  if (rows == 0 || cols == 0)
    return 0;
  if (!src || !dst || blockX == 0 || blockY == 0 || unroll == 0 ||
      blockX * blockY > 1024) {
    dev->report("hcamdLaunchCopy2DTiled: invalid argument");
    return 1;
  }
  const std::string name = std::string("hcamd_copy2d_tiled_") + suffix;
  Kernel *k = builtinKernel(dev, "copy", name.c_str());
  if (!k)
    return 1;
  int64_t u = (int64_t)unroll, s0 = ss0, d0 = ds0, r = (int64_t)rows,
          c = (int64_t)cols;
  void *args[] = {&u, &s0, &src, &r, &c, &d0, &dst};
  const size_t grid[3] = {ceilDiv(cols, blockX * unroll), ceilDiv(rows, blockY),
                          1};
  const size_t block[3] = {blockX, blockY, 1};
  return launch(queue, k, grid, block, args, 0);
}

int hcamdLaunchAddF32(OlQueue q, const float *a, const float *b, float *c,
                      size_t n) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  if (n == 0)
    return 0;
  if (!a || !b || !c) {
    queue->device->report("hcamdLaunchAddF32: null pointer");
    return 1;
  }
  void *args[] = {&a, &b, &c, &n};
  const int variant = variantOf("add");
  if (!(aligned16(a) && aligned16(b) && aligned16(c)) || variant == 9)
    return launch1d(queue, "elementwise", "hcamd_add_f32_scalar",
                    ceilDiv(n, 256), 256, args);
  static const char *const names[] = {
      "hcamd_add_f32_v4_nt", "hcamd_add_f32_v1",    "hcamd_add_f32_v2",
      "hcamd_add_f32_v4",    "hcamd_add_f32_v8",    "hcamd_add_f32_v1_nt",
      "hcamd_add_f32_v2_nt", "hcamd_add_f32_v4_nt", "hcamd_add_f32_v8_nt"};
  static const int vpt[] = {4, 1, 2, 4, 8, 1, 2, 4, 8};
  const int v = (variant >= 0 && variant <= 8) ? variant : 0;
  const size_t words = ceilDiv(n, 4);
  return launch1d(queue, "elementwise", names[v],
                  ceilDiv(words, 256 * (size_t)vpt[v]), 256, args);
}

int hcamdLaunchFmaF16(OlQueue q, const void *a, size_t lda, const void *b,
                      size_t ldb, const void *c, size_t ldc, void *d,
                      size_t ldd, size_t rows, size_t cols) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  if (rows == 0 || cols == 0)
    return 0;
  if (!a || !b || !c || !d) {
    dev->report("hcamdLaunchFmaF16: null pointer");
    return 1;
  }
  if (rows > 1 && (lda < cols || ldb < cols || ldc < cols || ldd < cols)) {
    dev->report("hcamdLaunchFmaF16: leading dimension smaller than cols");
    return 1;
  }
  const bool dense = rows == 1 || (lda == cols && ldb == cols && ldc == cols &&
                                   ldd == cols);
  const int variant = variantOf("fma");
  if (dense && aligned16(a) && aligned16(b) && aligned16(c) && aligned16(d) &&
      variant != 7) {
    // 0: the paced kernel (four waves per SIMD, a pause before the store);
    // 8..12: the same with other paces, for measurement
    static const char *const names[] = {
        "hcamd_fma_f16_v1_nt_w4_d6", "hcamd_fma_f16_v1",    "hcamd_fma_f16_v2",
        "hcamd_fma_f16_v4",          "hcamd_fma_f16_v1_nt", "hcamd_fma_f16_v2_nt",
        "hcamd_fma_f16_v4_nt",       nullptr,               "hcamd_fma_f16_v1_nt_w4_d0",
        "hcamd_fma_f16_v1_nt_w4_d3", "hcamd_fma_f16_v1_nt_w4_d12", "hcamd_fma_f16_v1_nt_w5_d12",
        "hcamd_fma_f16_v1_nt_w6_d8"};
    static const int vpt[] = {1, 1, 2, 4, 1, 2, 4, 0, 1, 1, 1, 1, 1};
    const int v = (variant >= 0 && variant <= 12) ? variant : 0;
    size_t n = rows * cols;
    const size_t words = ceilDiv(n, 8);
    void *args[] = {&a, &b, &c, &d, &n};
    return launch1d(queue, "elementwise", names[v],
                    ceilDiv(words, 256 * (size_t)vpt[v]), 256, args);
  }
  // windows: the widest access all four arrays' rows are aligned for
  size_t width = 1; // elements per access
  if (variant != 7) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                           reinterpret_cast<uintptr_t>(c) | reinterpret_cast<uintptr_t>(d) |
                           (rows > 1 ? (lda | ldb | ldc | ldd) * 2 : 0);
    width = bits % 16 == 0 ? 8 : bits % 8 == 0 ? 4 : bits % 4 == 0 ? 2 : 1;
  }
  Kernel *k = builtinKernel(dev, "elementwise",
                            width == 8   ? "hcamd_fma_f16_rows_v8"
                            : width == 4 ? "hcamd_fma_f16_rows_v4"
                            : width == 2 ? "hcamd_fma_f16_rows_v2"
                                         : "hcamd_fma_f16_2d");
  if (!k)
    return 1;
  // lanes per row: one per group of `width` elements plus one per leftover
  const size_t lanes = cols / width + cols % width;
  for (size_t r0 = 0; r0 < rows; r0 += 65535) {
    size_t nr = std::min(rows - r0, (size_t)65535);
    const char *pa = static_cast<const char *>(a) + r0 * lda * 2;
    const char *pb = static_cast<const char *>(b) + r0 * ldb * 2;
    const char *pc = static_cast<const char *>(c) + r0 * ldc * 2;
    char *pd = static_cast<char *>(d) + r0 * ldd * 2;
    void *args[] = {&pa, &lda, &pb, &ldb, &pc, &ldc, &pd, &ldd, &nr, &cols};
    const size_t grid[3] = {ceilDiv(lanes, 256), nr, 1};
    const size_t block[3] = {256, 1, 1};
    if (launch(queue, k, grid, block, args, 0))
      return 1;
  }
  return 0;
}

// ---------------------------------------------------------------------------
// Fused elementwise map (kernels/map.hip)
// ---------------------------------------------------------------------------
namespace {
constexpr size_t kMapMaxIn = HCAMD_MAP_MAX_INPUTS;
constexpr size_t kMapMaxProg = HCAMD_MAP_MAX_INSTRS;
constexpr int kMapDepth = HCAMD_MAP_STACK_DEPTH;

// Kernel argument block; layout shared with kernels/map.hip.
struct MapArgs {
  const void *in[kMapMaxIn];
  void *out;
  size_t ld[kMapMaxIn];
  size_t ldo;
  size_t rows, cols;
  uint32_t f16_mask;
  uint32_t n_instr;
  HcamdMapInstr prog[kMapMaxProg];
};

// Stack effect of an opcode: pops, pushes; -1 pops = unknown opcode.
void mapStackEffect(unsigned op, int &pops, int &pushes) {
  if (op == HCAMD_MAP_IN || op == HCAMD_MAP_CONST) {
    pops = 0, pushes = 1;
  } else if (op >= HCAMD_MAP_ADD && op <= HCAMD_MAP_RDIV) {
    pops = 2, pushes = 1;
  } else if (op >= HCAMD_MAP_ADDI && op <= HCAMD_MAP_RDIV_IN) {
    pops = 1, pushes = 1;
  } else {
    pops = -1, pushes = 0;
  }
}
// The same with the masked-division forms, which only the element-wise map and
// its sum take.
void mapStackEffectMasked(unsigned op, int &pops, int &pushes) {
  if (op == HCAMD_MAP_MDIV || op == HCAMD_MAP_RMDIV)
    pops = 2, pushes = 1;
  else if (op >= HCAMD_MAP_MDIVI && op <= HCAMD_MAP_MLOG)
    pops = 1, pushes = 1;
  else
    mapStackEffect(op, pops, pushes);
}
} // namespace

namespace {
// Shared by the map and the map-sum entry points.  `sum`: out is the fp32 cell
// the sum of all results is added to; outType and ldo are not used.
int launchMap(OlQueue q, bool sum, const HcamdMapInstr *prog, size_t nInstr,
              const void *const *inputs, const int *inputTypes,
              const size_t *inputLd, size_t nInputs, void *out, int outType,
              size_t ldo, size_t rows, size_t cols) {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *who = sum ? "hcamdLaunchMapSum" : "hcamdLaunchMap";
  if (!prog || nInstr == 0 || nInstr > kMapMaxProg) {
    dev->report("%s: program of %zu instructions (1..%zu allowed)", who,
                nInstr, kMapMaxProg);
    return 1;
  }
  if (nInputs > kMapMaxIn || (nInputs && (!inputs || !inputTypes || !inputLd))) {
    dev->report("%s: %zu operands (at most %zu)", who, nInputs,
                kMapMaxIn);
    return 1;
  }
  auto typeOk = [](int t) { return t == HCAMD_F32 || t == HCAMD_F16; };
  if (!typeOk(outType)) {
    dev->report("%s: unsupported output type %d", who, outType);
    return 1;
  }
  // The program must keep the stack within bounds and leave one value.
  int sp = 0;
  bool hasMasked = false; // numpy.ma's division forms: only the element-wise kernels have them
  for (size_t i = 0; i < nInstr; ++i) {
    int pops, pushes;
    mapStackEffectMasked(prog[i].op, pops, pushes);
    if (pops < 0) {
      dev->report("%s: unknown opcode %u at %zu", who, prog[i].op, i);
      return 1;
    }
    const bool maskedOperand = prog[i].op == HCAMD_MAP_MDIV_IN || prog[i].op == HCAMD_MAP_RMDIV_IN;
    hasMasked = hasMasked || (prog[i].op >= HCAMD_MAP_MDIV && prog[i].op <= HCAMD_MAP_MLOG);
    const bool readsOperand =
        prog[i].op == HCAMD_MAP_IN || maskedOperand ||
        (prog[i].op >= HCAMD_MAP_ADD_IN && prog[i].op <= HCAMD_MAP_RDIV_IN);
    if (readsOperand && (maskedOperand ? prog[i].arg & 0xffu : prog[i].arg) >= nInputs) {
      dev->report("%s: operand %u at %zu (only %zu given)", who,
                  prog[i].arg, i, nInputs);
      return 1;
    }
    if (sp < pops) {
      dev->report("%s: stack underflow at %zu", who, i);
      return 1;
    }
    sp += pushes - pops;
    if (sp > kMapDepth) {
      dev->report("%s: stack deeper than %d at %zu", who, kMapDepth, i);
      return 1;
    }
  }
  if (sp != 1) {
    dev->report("%s: program leaves %d values, expected 1", who, sp);
    return 1;
  }
  if (rows == 0 || cols == 0)
    return 0;
  if (!out) {
    dev->report("%s: null pointer", who);
    return 1;
  }
  MapArgs a{};
  bool dense = sum || rows == 1 || ldo == cols;
  bool aligned = sum || aligned16(out);
  if (!sum && rows > 1 && ldo < cols) {
    dev->report("%s: leading dimension smaller than cols", who);
    return 1;
  }
  for (size_t i = 0; i < nInputs; ++i) {
    if (!inputs[i]) {
      dev->report("%s: null pointer", who);
      return 1;
    }
    if (!typeOk(inputTypes[i])) {
      dev->report("%s: unsupported operand type %d", who, inputTypes[i]);
      return 1;
    }
    if (rows > 1 && inputLd[i] < cols) {
      dev->report("%s: leading dimension smaller than cols", who);
      return 1;
    }
    a.in[i] = inputs[i];
    a.ld[i] = inputLd[i];
    if (inputTypes[i] == HCAMD_F16)
      a.f16_mask |= 1u << i;
    dense = dense && (rows == 1 || inputLd[i] == cols);
    aligned = aligned && aligned16(inputs[i]);
  }
  if (outType == HCAMD_F16)
    a.f16_mask |= 1u << 8;
  a.out = out;
  a.ldo = ldo;
  a.n_instr = static_cast<uint32_t>(nInstr);
  std::memcpy(a.prog, prog, nInstr * sizeof(HcamdMapInstr));
  uint32_t nIn = static_cast<uint32_t>(nInputs);
  void *args[] = {&a, &nIn};
  constexpr size_t kPerGroup = 256 * 8; // elements per workgroup: eight per lane
  if (dense && aligned && variantOf("map") != 1) {
    a.rows = 1;
    a.cols = rows * cols;
    // The reduction picks its kernel by operand count and storage type: fewer
    // or narrower operands leave registers for more chunks in flight per lane.
    const bool half = nInputs > 0 && (a.f16_mask & 0xffu) == (1u << nInputs) - 1u;
    // sum(x) and sum(x * y) over fp32 have kernels of their own (variant 2 of
    // "map" keeps them on the interpreter)
    if (sum && (a.f16_mask & 0xffu) == 0 && variantOf("map") != 2) {
      const bool isSum = nInstr == 1 && prog[0].op == HCAMD_MAP_IN;
      const bool isDot = nInstr == 2 && prog[0].op == HCAMD_MAP_IN &&
                         prog[1].op == HCAMD_MAP_MUL_IN;
      if (isSum || isDot) {
        const void *x = inputs[prog[0].arg];
        const void *y = isDot ? inputs[prog[1].arg] : x;
        size_t n = a.cols;
        void *rargs[4];
        int na = 0;
        rargs[na++] = &x;
        if (isDot)
          rargs[na++] = &y;
        rargs[na++] = &out;
        rargs[na++] = &n;
        const size_t groups = std::min(std::max(ceilDiv(n, (size_t)1024 * 16), (size_t)1),
                                       (size_t)computeUnitsOf(dev));
        return launch1d(queue, "map", isDot ? "hcamd_dot_f32" : "hcamd_sum_f32",
                        groups, 1024, rargs);
      }
    }
    const char *name = "hcamd_map_flat";
    size_t u = 1;
    if (sum && half) {
      name = nInputs <= 2 ? "hcamd_map_sum_flat_n2u4h" : "hcamd_map_sum_flat_n4u2h";
      u = nInputs <= 2 ? 4 : 2;
    } else if (sum && nInputs <= 1) {
      name = "hcamd_map_sum_flat_n1u4";
      u = 4;
    } else if (sum && nInputs <= 2) {
      name = "hcamd_map_sum_flat_n2u2";
      u = 2;
    } else if (sum) {
      name = "hcamd_map_sum_flat_n4u1";
    } else if (half && outType == HCAMD_F16 && nInputs <= 2 && variantOf("map") != 3) {
      name = "hcamd_map_flat_n2u4h"; // (variant 3 of "map": one chunk per lane whatever the operands)
      u = 4;
    }
    // A chain (an operand or a constant first, then only operations that change
    // the value in place) of five instructions or more runs on the chain
    // interpreter, sixteen elements of a lane to a dispatch (variant 4 of "map":
    // every chain; 5: none).
    if (!sum && a.cols >= 4096 && variantOf("map") != 5 && variantOf("map") != 3 &&
        (nInstr >= 5 || variantOf("map") == 4)) {
      bool chain = prog[0].op == HCAMD_MAP_IN || prog[0].op == HCAMD_MAP_CONST;
      for (size_t pc = 1; pc < nInstr && chain; ++pc)
        chain = !(prog[pc].op <= HCAMD_MAP_RDIV || prog[pc].op == HCAMD_MAP_MDIV ||
                  prog[pc].op == HCAMD_MAP_RMDIV);
      if (chain) {
        const bool allHalf = half && outType == HCAMD_F16;
        const char *chainName = nInputs <= 2 ? (allHalf ? "hcamd_map_chain_n2h" : "hcamd_map_chain_n2")
                                             : (allHalf ? "hcamd_map_chain_n4h" : "hcamd_map_chain_n4");
        return launch1d(queue, "map", chainName, a.cols / 4096 + (a.cols % 4096 ? 1 : 0), 256, args);
      }
    }
    // the reduction: 1024-lane workgroups, one per CU, each striding over the
    // vector and ending in one atomic addition
    const size_t threads = sum ? 1024 : 256;
    size_t groups = std::max(ceilDiv(a.cols, threads * 8 * u), (size_t)1);
    if (sum)
      groups = std::min(groups, (size_t)computeUnitsOf(dev));
    return launch1d(queue, "map", name, groups, threads, args);
  }
  a.cols = cols;
  // Windows whose rows all start on 16-byte boundaries: 16-byte accesses along
  // the rows (variant 1 of "map" keeps the element-wise kernel below).
  bool rowsAligned = variantOf("map") != 1 &&
                     (sum || (aligned16(out) && (ldo * (outType == HCAMD_F16 ? 2 : 4)) % 16 == 0));
  for (size_t i = 0; i < nInputs && rowsAligned; ++i)
    rowsAligned = aligned16(inputs[i]) &&
                  (inputLd[i] * (inputTypes[i] == HCAMD_F16 ? 2 : 4)) % 16 == 0;
  const size_t perRow = cols / 8 + (cols % 8 ? 1 : 0);
  if (rowsAligned && rows <= ((size_t)1 << 30) / perRow) {
    a.rows = rows;
    const size_t items = rows * perRow;
    const size_t threads = sum ? 1024 : 256;
    size_t groups = ceilDiv(items, threads);
    if (sum)
      groups = std::min(groups, (size_t)computeUnitsOf(dev));
    return launch1d(queue, "map", sum ? "hcamd_map_sum_rows" : "hcamd_map_rows", groups,
                    threads, args);
  }
  // Windows with fp16 operands whose rows are not 16-byte aligned: the row-program
  // kernel run as a single store stage reads them coalesced with 32-bit index
  // arithmetic, about twice as fast as the element-wise kernel below, which
  // stays for fp32 (where it is the faster one) and under variant 1 of "map".
  if (!sum && a.f16_mask != 0 && variantOf("map") != 1 && !hasMasked) {
    const HcamdRowStage whole = {HCAMD_ROW_STORE, static_cast<uint32_t>(nInstr), 0};
    return hcamdLaunchRowProgram(q, prog, &whole, 1, inputs, inputTypes, inputLd, nInputs,
                                 nullptr, nullptr, 0, out, outType, ldo, rows, cols);
  }
  Kernel *k = builtinKernel(dev, "map",
                            sum ? "hcamd_map_sum_strided" : "hcamd_map_strided");
  if (!k)
    return 1;
  const size_t esz_out = outType == HCAMD_F16 ? 2 : 4;
  if (sum) {
    a.rows = rows;
    const size_t groups = std::min(rows * ceilDiv(cols, kPerGroup),
                                   (size_t)computeUnitsOf(dev) * 4);
    const size_t grid[3] = {groups, 1, 1}, block[3] = {256, 1, 1};
    return launch(queue, k, grid, block, args, 0);
  }
  for (size_t r0 = 0; r0 < rows; r0 += 65535) {
    const size_t nr = std::min(rows - r0, (size_t)65535);
    a.rows = nr;
    for (size_t i = 0; i < nInputs; ++i)
      a.in[i] = static_cast<const char *>(inputs[i]) +
                r0 * inputLd[i] * (inputTypes[i] == HCAMD_F16 ? 2 : 4);
    a.out = sum ? out : static_cast<char *>(out) + r0 * ldo * esz_out;
    const size_t grid[3] = {ceilDiv(cols, kPerGroup), nr, 1};
    const size_t block[3] = {256, 1, 1};
    if (launch(queue, k, grid, block, args, 0))
      return 1;
  }
  return 0;
}
} // namespace

int hcamdLaunchMap(OlQueue q, const HcamdMapInstr *prog, size_t nInstr,
                   const void *const *inputs, const int *inputTypes,
                   const size_t *inputLd, size_t nInputs, void *out,
                   int outType, size_t ldo, size_t rows,
                   size_t cols) noexcept {
  return launchMap(q, false, prog, nInstr, inputs, inputTypes, inputLd, nInputs,
                   out, outType, ldo, rows, cols);
}

namespace {
struct IMapInstr {
  uint16_t op, arg;
  int32_t imm;
};
struct IMapArgs {
  const void *in[4];
  void *out;
  size_t ld[4];
  size_t ldo, rows, cols;
  uint32_t out_u8, vec, n_instr;
  IMapInstr prog[32];
};
} // namespace

int hcamdLaunchIMap(OlQueue q, const HcamdMapInstr *prog, size_t nInstr,
                    const void *const *inputs, const size_t *inputLd, size_t nInputs,
                    void *out, int outType, size_t ldo, size_t rows, size_t cols) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *who = "hcamdLaunchIMap";
  if (!prog || nInstr == 0 || nInstr > 32) {
    dev->report("%s: program of %zu instructions (1..32)", who, nInstr);
    return 1;
  }
  if (nInputs > 4 || (nInputs && (!inputs || !inputLd)) || !out) {
    dev->report("%s: %zu operands (0..4) or a null pointer", who, nInputs);
    return 1;
  }
  if (outType != HCAMD_I32 && outType != HCAMD_U8) {
    dev->report("%s: unsupported output type %d", who, outType);
    return 1;
  }
  IMapArgs a{};
  int sp = 0;
  for (size_t i = 0; i < nInstr; ++i) {
    const unsigned op = prog[i].op;
    if (op == HCAMD_IMAP_END || op >= HCAMD_IMAP_COUNT) {
      dev->report("%s: bad opcode %u at %zu", who, op, i);
      return 1;
    }
    if (op == HCAMD_IMAP_IN && prog[i].arg >= nInputs) {
      dev->report("%s: operand %u at %zu (only %zu given)", who, prog[i].arg, i, nInputs);
      return 1;
    }
    const bool push = op == HCAMD_IMAP_IN || op == HCAMD_IMAP_CONST;
    const bool select = op == HCAMD_IMAP_SELECT; // three entries in, one out
    const bool unary = op >= HCAMD_IMAP_NEG && !select;
    if (sp < (push ? 0 : unary ? 1 : select ? 3 : 2)) {
      dev->report("%s: stack underflow at %zu", who, i);
      return 1;
    }
    sp += push ? 1 : unary ? 0 : select ? -2 : -1;
    if (sp > 4) {
      dev->report("%s: stack deeper than 4 at %zu", who, i);
      return 1;
    }
    a.prog[i].op = prog[i].op;
    a.prog[i].arg = prog[i].arg;
    std::memcpy(&a.prog[i].imm, &prog[i].imm, sizeof(int32_t));
  }
  if (sp != 1) {
    dev->report("%s: program leaves %d values, expected 1", who, sp);
    return 1;
  }
  if (rows == 0 || cols == 0)
    return 0;
  if (rows > 65535 && cols == 1) { // a column vector: walk it as one row when it is dense
    bool dense = ldo == 1;
    for (size_t i = 0; i < nInputs; ++i)
      dense = dense && inputLd[i] == 1;
    if (dense) {
      cols = rows;
      rows = 1;
    }
  }
  bool vec = outType == HCAMD_I32 && aligned16(out) && (rows == 1 || ldo % 4 == 0);
  for (size_t i = 0; i < nInputs; ++i) {
    if (!inputs[i]) {
      dev->report("%s: null pointer", who);
      return 1;
    }
    if (rows > 1 && inputLd[i] < cols) {
      dev->report("%s: leading dimension smaller than cols", who);
      return 1;
    }
    a.in[i] = inputs[i];
    a.ld[i] = inputLd[i];
    vec = vec && aligned16(inputs[i]) && (rows == 1 || inputLd[i] % 4 == 0);
  }
  if (rows > 1 && ldo < cols) {
    dev->report("%s: leading dimension smaller than cols", who);
    return 1;
  }
  a.out = out;
  a.ldo = ldo;
  a.rows = rows;
  a.cols = cols;
  a.out_u8 = outType == HCAMD_U8 ? 1u : 0u;
  a.vec = vec ? 1u : 0u;
  a.n_instr = (uint32_t)nInstr;
  Kernel *k = builtinKernel(dev, "imap", "hcamd_imap_i32");
  if (!k)
    return 1;
  void *args[] = {&a};
  const size_t block[3] = {256, 1, 1};
  // blockIdx.y numbers the rows: at most 65535 of them per launch
  for (size_t r0 = 0; r0 < rows; r0 += 65535) {
    const size_t nr = std::min(rows - r0, (size_t)65535);
    a.rows = nr;
    for (size_t i = 0; i < nInputs; ++i)
      a.in[i] = static_cast<const char *>(inputs[i]) + r0 * inputLd[i] * sizeof(int32_t);
    a.out = static_cast<char *>(out) + r0 * ldo * (outType == HCAMD_U8 ? 1 : sizeof(int32_t));
    const size_t grid[3] = {ceilDiv(ceilDiv(cols, (size_t)4), (size_t)256), nr, 1};
    if (int rc = launch(queue, k, grid, block, args, 0))
      return rc;
  }
  return 0;
}

namespace {
// Argument block of hcamd_fmap (device layout).
struct FMapArgs {
  const void *in[4];
  void *out;
  size_t ld[4];
  size_t ldo, rows, cols;
  uint32_t f16_mask, out_type, vec, store_all, n_instr;
  HcamdMapInstr prog[48];
};
} // namespace

int hcamdLaunchFMap(OlQueue q, const HcamdMapInstr *prog, size_t nInstr,
                    const void *const *inputs, const int *inputTypes, const size_t *inputLd,
                    size_t nInputs, void *out, int outType, size_t ldo, size_t rows,
                    size_t cols, int storeAll) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *who = "hcamdLaunchFMap";
  if (!prog || nInstr == 0 || nInstr > 48) {
    dev->report("%s: program of %zu instructions (1..48)", who, nInstr);
    return 1;
  }
  if (nInputs > 4 || (nInputs && (!inputs || !inputLd || !inputTypes)) || !out) {
    dev->report("%s: %zu operands (0..4) or a null pointer", who, nInputs);
    return 1;
  }
  if (outType != HCAMD_F32 && outType != HCAMD_F16 && outType != HCAMD_U8) {
    dev->report("%s: unsupported output type %d", who, outType);
    return 1;
  }
  FMapArgs a{};
  int sp = 0;
  for (size_t i = 0; i < nInstr; ++i) {
    const unsigned op = prog[i].op;
    if (op == HCAMD_FMAP_END || op >= HCAMD_FMAP_COUNT) {
      dev->report("%s: bad opcode %u at %zu", who, op, i);
      return 1;
    }
    if (op == HCAMD_FMAP_IN && prog[i].arg >= nInputs) {
      dev->report("%s: operand %u at %zu (only %zu given)", who, prog[i].arg, i, nInputs);
      return 1;
    }
    const bool push = op == HCAMD_FMAP_IN || op == HCAMD_FMAP_CONST;
    const bool select = op == HCAMD_FMAP_SELECT; // three entries in, one out
    const bool unary = op >= HCAMD_FMAP_NEG && !select && op != HCAMD_FMAP_MERGE; // (MERGE: two in, one out)
    if (sp < (push ? 0 : unary ? 1 : select ? 3 : 2)) {
      dev->report("%s: stack underflow at %zu", who, i);
      return 1;
    }
    sp += push ? 1 : unary ? 0 : select ? -2 : -1;
    if (sp > 4) {
      dev->report("%s: stack deeper than 4 at %zu", who, i);
      return 1;
    }
    a.prog[i] = prog[i];
  }
  if (sp != 1) {
    dev->report("%s: program leaves %d values, expected 1", who, sp);
    return 1;
  }
  if (rows == 0 || cols == 0)
    return 0;
  if (rows > 65535 && cols == 1) { // a column vector: walk it as one row when it is dense
    bool dense = ldo == 1;
    for (size_t i = 0; i < nInputs; ++i)
      dense = dense && inputLd[i] == 1;
    if (dense) {
      cols = rows;
      rows = 1;
    }
  }
  // a row of four-element pieces: fp32 pieces are 16 bytes, fp16 pieces 8
  auto piece_ok = [&](const void *p, int type, size_t ld) {
    const size_t bytes = type == HCAMD_F16 ? 8 : 16;
    return reinterpret_cast<uintptr_t>(p) % bytes == 0 && (rows == 1 || ld % 4 == 0);
  };
  bool vec = outType == HCAMD_U8 || piece_ok(out, outType, ldo);
  for (size_t i = 0; i < nInputs; ++i) {
    if (!inputs[i]) {
      dev->report("%s: null pointer", who);
      return 1;
    }
    if (inputTypes[i] != HCAMD_F32 && inputTypes[i] != HCAMD_F16 && inputTypes[i] != HCAMD_I32) {
      dev->report("%s: unsupported operand type %d", who, inputTypes[i]);
      return 1;
    }
    if (rows > 1 && inputLd[i] < cols) {
      dev->report("%s: leading dimension smaller than cols", who);
      return 1;
    }
    a.in[i] = inputs[i];
    a.ld[i] = inputLd[i];
    if (inputTypes[i] == HCAMD_F16)
      a.f16_mask |= 1u << i;
    if (inputTypes[i] == HCAMD_I32)
      a.f16_mask |= 1u << (8 + i); // converted to fp32 when read
    vec = vec && piece_ok(inputs[i], inputTypes[i], inputLd[i]);
  }
  if (rows > 1 && ldo < cols) {
    dev->report("%s: leading dimension smaller than cols", who);
    return 1;
  }
  a.out = out;
  a.ldo = ldo;
  a.rows = rows;
  a.cols = cols;
  a.out_type = outType == HCAMD_F32 ? 0u : outType == HCAMD_F16 ? 1u : 2u;
  a.vec = vec ? 1u : 0u;
  a.store_all = storeAll ? 1u : 0u;
  a.n_instr = (uint32_t)nInstr;
  // eight elements of a lane to a dispatch where the rows are long enough to
  // give a workgroup its 2048 and move in whole pieces
  const size_t perLane = vec && cols >= 2048 ? 8 : 4;
  Kernel *k = builtinKernel(dev, "fmap", perLane == 8 ? "hcamd_fmap_v8" : "hcamd_fmap");
  if (!k)
    return 1;
  void *args[] = {&a};
  const size_t block[3] = {256, 1, 1};
  const size_t outSize = outType == HCAMD_F32 ? 4 : outType == HCAMD_F16 ? 2 : 1;
  // blockIdx.y numbers the rows: at most 65535 of them per launch
  for (size_t r0 = 0; r0 < rows; r0 += 65535) {
    const size_t nr = std::min(rows - r0, (size_t)65535);
    a.rows = nr;
    for (size_t i = 0; i < nInputs; ++i)
      a.in[i] = static_cast<const char *>(inputs[i]) +
                r0 * inputLd[i] * (inputTypes[i] == HCAMD_F16 ? 2 : 4);
    a.out = static_cast<char *>(out) + r0 * ldo * outSize;
    const size_t grid[3] = {ceilDiv(ceilDiv(cols, perLane), (size_t)256), nr, 1};
    if (int rc = launch(queue, k, grid, block, args, 0))
      return rc;
  }
  return 0;
}

int hcamdLaunchMapSum(OlQueue q, const HcamdMapInstr *prog, size_t nInstr,
                      const void *const *inputs, const int *inputTypes,
                      const size_t *inputLd, size_t nInputs, float *cell,
                      size_t rows, size_t cols) noexcept {
  return launchMap(q, true, prog, nInstr, inputs, inputTypes, inputLd, nInputs,
                   cell, HCAMD_F32, cols, rows, cols);
}

namespace {
// Second argument block of the column-reduction kernels (device layout).
struct ColArgs {
  float *partial;
  uint32_t colsPad, band, kind, lanes, interleaved, outVec, nPost, masked;
  uint32_t fillEmpty; // the finishing launch: a maximum / minimum over no active element is 1e20
  HcamdMapInstr post[HCAMD_COLS_MAX_POST];
};

// Stack discipline of a map program: within bounds, one value left, operands
// below nInputs.
bool mapProgramOk(Device *dev, const char *who, const HcamdMapInstr *prog, size_t nInstr,
                  size_t nInputs, bool allowMasked = false) {
  int sp = 0;
  for (size_t i = 0; i < nInstr; ++i) {
    int pops, pushes;
    if (allowMasked)
      mapStackEffectMasked(prog[i].op, pops, pushes);
    else
      mapStackEffect(prog[i].op, pops, pushes);
    if (pops < 0) {
      dev->report("%s: unknown opcode %u at %zu", who, prog[i].op, i);
      return false;
    }
    const bool readsOperand =
        prog[i].op == HCAMD_MAP_IN ||
        (prog[i].op >= HCAMD_MAP_ADD_IN && prog[i].op <= HCAMD_MAP_RDIV_IN);
    if (readsOperand && prog[i].arg >= nInputs) {
      dev->report("%s: operand %u at %zu (only %zu given)", who, prog[i].arg, i, nInputs);
      return false;
    }
    if (sp < pops) {
      dev->report("%s: stack underflow at %zu", who, i);
      return false;
    }
    sp += pushes - pops;
    if (sp > kMapDepth) {
      dev->report("%s: stack deeper than %d at %zu", who, kMapDepth, i);
      return false;
    }
  }
  if (sp != 1) {
    dev->report("%s: program leaves %d values, expected 1", who, sp);
    return false;
  }
  return true;
}

// Lanes that share a row: 64, or the next power of two above the chunks of a
// narrow row.
size_t colLanes(size_t cols) {
  const size_t perRow = ceilDiv(cols, (size_t)8);
  size_t lanes = 1;
  while (lanes < 64 && lanes < perRow)
    lanes *= 2;
  return lanes;
}

// Bands of rows a column reduction is cut into, so that the launch has a few
// workgroups per compute unit however narrow the window is; 1 = one launch.
void colBands(size_t rows, size_t cols, size_t &bands, size_t &band) {
  const size_t lanes = colLanes(cols);
  const size_t blocks = ceilDiv(ceilDiv(cols, (size_t)8), lanes);
  const size_t turn = 16 * (64 / lanes); // rows of one turn of 4 waves x 4 rows in flight
  const size_t wanted = ceilDiv((size_t)1536, blocks); // six workgroups for each of 256 compute units
  bands = std::max(std::min(wanted, rows / (4 * turn)), (size_t)1);
  band = ceilDiv(ceilDiv(rows, bands), turn) * turn;
  bands = ceilDiv(rows, band);
}

// The sums of x and of x * x over a dense fp32 window have band kernels of their
// own (hcamd_cols_sum_f32, hcamd_cols_sumsq_f32), which run fastest with many
// short bands: about sixteen workgroups of sixteen waves for each compute
// unit, 32 rows or more to a band (root mean square down 4096 x 8192, both
// launches: bands of 32 rows 24.1 us, of 64 rows 27.0 us; the partial sums are
// then 1/32 of the window).
bool colDenseShape(size_t cols) { return cols % 8 == 0 && cols >= 256; }
void colBandsDense(size_t rows, size_t cols, size_t &bands, size_t &band) {
  const size_t blocks = ceilDiv(cols, (size_t)256);
  const size_t wanted = ceilDiv((size_t)4096, blocks);
  bands = std::max(std::min(wanted, rows / 32), (size_t)1);
  band = ceilDiv(ceilDiv(rows, bands), (size_t)32) * 32;
  bands = ceilDiv(rows, band);
}

// The bands of the first launch are the rows of the second, which always
// finishes: it spreads its few rows over the lanes of a wave (fewer lanes per
// row), so that a wave has them all in flight in one or two turns.
size_t colSecondLanes(size_t bands, size_t lanes) {
  while (lanes > 1 && ceilDiv(bands, 16 * (64 / lanes)) > 1)
    lanes /= 2;
  return lanes;
}
} // namespace

size_t hcamdMapReduceColsWorkspace(size_t rows, size_t cols) noexcept {
  if (rows == 0 || cols == 0)
    return 0;
  size_t bands, band;
  colBands(rows, cols, bands, band);
  if (bands > 1 && colDenseShape(cols)) {
    // (whichever kernel the program gets: the caller sizes the workspace by the shape alone)
    size_t denseBands, denseBand;
    colBandsDense(rows, cols, denseBands, denseBand);
    bands = std::max(bands, denseBands);
  }
  return bands > 1 ? bands * ceilDiv(cols, (size_t)8) * 8 * sizeof(float) : 0;
}

int hcamdLaunchMapReduceCols(OlQueue q, int kind, const HcamdMapInstr *prog, size_t nInstr,
                             const HcamdMapInstr *post, size_t nPost,
                             const void *const *inputs, const int *inputTypes,
                             const size_t *inputLd, size_t nInputs, void *out, int outType,
                             size_t rows, size_t cols, void *workspace,
                             size_t workspaceBytes) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *who = "hcamdLaunchMapReduceCols";
  if (kind != HCAMD_COLS_SUM && kind != HCAMD_COLS_MAX && kind != HCAMD_COLS_MIN) {
    dev->report("%s: unknown reduction %d", who, kind);
    return 1;
  }
  if (!prog || nInstr == 0 || nInstr > kMapMaxProg || nPost > HCAMD_COLS_MAX_POST ||
      (nPost && !post)) {
    dev->report("%s: programs of %zu and %zu instructions (1..%zu and 0..%d allowed)", who,
                nInstr, nPost, kMapMaxProg, HCAMD_COLS_MAX_POST);
    return 1;
  }
  if (nInputs == 0 || nInputs > kMapMaxIn || !inputs || !inputTypes || !inputLd) {
    dev->report("%s: %zu operands (1..%zu)", who, nInputs, kMapMaxIn);
    return 1;
  }
  auto typeOk = [](int t) { return t == HCAMD_F32 || t == HCAMD_F16; };
  if (!typeOk(outType)) {
    dev->report("%s: unsupported output type %d", who, outType);
    return 1;
  }
  if (!mapProgramOk(dev, who, prog, nInstr, nInputs, true) ||
      (nPost && !mapProgramOk(dev, who, post, nPost, 1, true)))
    return 1;
  if (cols == 0)
    return 0;
  if (rows == 0) {
    dev->report("%s: no rows to reduce", who);
    return 1;
  }
  if (rows >= ((size_t)1 << 32) || cols > ((size_t)1 << 32) - 1024) {
    dev->report("%s: window of %zu x %zu (below 2^32 each)", who, rows, cols);
    return 1;
  }
  if (!out) {
    dev->report("%s: null pointer", who);
    return 1;
  }
  MapArgs a{};
  ColArgs c{};
  bool allVec = true;
  for (size_t i = 0; i < nInputs; ++i) {
    if (!inputs[i]) {
      dev->report("%s: null pointer", who);
      return 1;
    }
    if (!typeOk(inputTypes[i])) {
      dev->report("%s: unsupported operand type %d", who, inputTypes[i]);
      return 1;
    }
    // leading dimension 0: a vector of cols elements that every row uses
    if (inputLd[i] != 0 && rows > 1 && inputLd[i] < cols) {
      dev->report("%s: leading dimension smaller than cols", who);
      return 1;
    }
    a.in[i] = inputs[i];
    a.ld[i] = inputLd[i];
    const size_t size = inputTypes[i] == HCAMD_F16 ? 2 : 4;
    if (inputTypes[i] == HCAMD_F16)
      a.f16_mask |= 1u << i;
    allVec = allVec && aligned16(inputs[i]) && (inputLd[i] * size) % 16 == 0;
  }
  const size_t colsPad = ceilDiv(cols, (size_t)8) * 8;
  size_t bands, band;
  colBands(rows, cols, bands, band);
  // The sums of x and of x * x over a dense fp32 window at least a wave's 256
  // columns wide have a kernel of their own for the first launch (variant 1 of
  // "cols" keeps the general one): 4096 x 8192, both launches, 36.8 -> 32.7 us,
  // and 24.1 us with the shorter bands that kernel likes.
  const bool plain = nInstr == 1 && prog[0].op == HCAMD_MAP_IN;
  const bool square = (nInstr == 3 && prog[0].op == HCAMD_MAP_IN && prog[1].op == HCAMD_MAP_IN &&
                       prog[2].op == HCAMD_MAP_MUL) ||
                      (nInstr == 2 && prog[0].op == HCAMD_MAP_IN && prog[1].op == HCAMD_MAP_MUL_IN);
  const bool denseSum = bands > 1 && (plain || square) && kind == HCAMD_COLS_SUM && nInputs == 1 &&
                        inputTypes[0] == HCAMD_F32 && inputLd[0] != 0 && allVec && colDenseShape(cols) &&
                        variantOf("cols") != 1;
  if (denseSum)
    colBandsDense(rows, cols, bands, band);
  const size_t floats = bands > 1 ? bands * colsPad : 0;
  if (floats && (!workspace || !aligned16(workspace) || workspaceBytes < floats * sizeof(float))) {
    dev->report("%s: workspace of %zu bytes, 16-byte aligned, needed (%zu given)", who,
                floats * sizeof(float), workspaceBytes);
    return 1;
  }
  auto launchOne = [&](MapArgs &ma, ColArgs &ca, size_t nIn, size_t nBands) {
    const char *name = nIn <= 1   ? "hcamd_map_reduce_cols_n1u4"
                       : nIn <= 2 ? "hcamd_map_reduce_cols_n2u2"
                                  : "hcamd_map_reduce_cols_n4u1";
    Kernel *k = builtinKernel(dev, "map", name);
    if (!k)
      return 1;
    uint32_t n = static_cast<uint32_t>(nIn);
    void *args[] = {&ma, &ca, &n};
    const size_t grid[3] = {ceilDiv(colsPad / 8, (size_t)ca.lanes), nBands, 1};
    const size_t block[3] = {256, 1, 1};
    return launch(queue, k, grid, block, args, 0);
  };
  // the launch that runs `post` and stores
  auto finishing = [&](MapArgs &ma, ColArgs &ca) {
    ma.out = out;
    if (outType == HCAMD_F16)
      ma.f16_mask |= 1u << 8;
    ca.outVec = aligned16(out) ? 1u : 0u;
    ca.nPost = static_cast<uint32_t>(nPost);
    if (nPost)
      std::memcpy(ca.post, post, nPost * sizeof(HcamdMapInstr));
    // numpy.ma's maximum / minimum of a column without an active element is
    // deactivated and holds its fill value, which is what a per-column result,
    // a bare numpy.ma array written in full, then stores.  (The fold's identity
    // stands for "no active element": a column whose active values are all
    // -inf (+inf) is taken for an empty one.)
    ca.fillEmpty = c.masked && kind != HCAMD_COLS_SUM ? 1u : 0u;
  };
  a.rows = rows;
  a.cols = cols;
  a.n_instr = static_cast<uint32_t>(nInstr);
  std::memcpy(a.prog, prog, nInstr * sizeof(HcamdMapInstr));
  c.kind = static_cast<uint32_t>(kind);
  for (size_t i = 0; i < nInstr; ++i)
    if (prog[i].op >= HCAMD_MAP_MDIV && prog[i].op <= HCAMD_MAP_MLOG && prog[i].op != HCAMD_MAP_CLEAR)
      c.masked = 1; // numpy.ma's forms: the folds leave inactive elements out
  c.colsPad = static_cast<uint32_t>(colsPad);
  c.band = static_cast<uint32_t>(band);
  c.lanes = static_cast<uint32_t>(colLanes(cols));
  c.interleaved = allVec ? 0u : 1u;
  if (bands == 1) {
    // few rows: fewer lanes to a row, as in the launch that folds bands
    c.lanes = static_cast<uint32_t>(colSecondLanes(rows, c.lanes));
    finishing(a, c);
    return launchOne(a, c, nInputs, 1);
  }
  c.partial = static_cast<float *>(workspace);
  if (denseSum) {
    // (variant 2: four waves to a workgroup with eight rows in flight each)
    const bool few = variantOf("cols") == 2;
    const size_t lanes = few ? 256 : 1024;
    char name[64];
    snprintf(name, sizeof name, "%s%s", square ? "hcamd_cols_sumsq_f32" : "hcamd_cols_sum_f32",
             few ? "_w4u8" : "");
    Kernel *k = builtinKernel(dev, "map", name);
    if (!k)
      return 1;
    const void *x = inputs[0];
    size_t ld = inputLd[0];
    float *partial = c.partial;
    uint32_t nCols = static_cast<uint32_t>(cols), pad = c.colsPad, nRows = static_cast<uint32_t>(rows),
             perBand = c.band;
    void *args[] = {&x, &ld, &partial, &nCols, &pad, &nRows, &perBand};
    const size_t grid[3] = {ceilDiv(cols, (size_t)256), bands, 1};
    const size_t block[3] = {lanes, 1, 1};
    if (int rc = launch(queue, k, grid, block, args, 0))
      return rc;
  } else if (int rc = launchOne(a, c, nInputs, bands)) {
    return rc;
  }
  // A sum whose post program only changes the folded value in place (the
  // division of a mean, the root of a norm) into a dense fp32 result: the bands
  // fold on a kernel that takes the program as arguments and interprets nothing.
  struct FoldPost {
    uint32_t n;
    uint32_t op[4];
    float imm[4];
  } fp{};
  bool simple = kind == HCAMD_COLS_SUM && outType == HCAMD_F32 && aligned16(out) && cols % 4 == 0 &&
                nPost <= 5 && variantOf("cols") != 1 &&
                (nPost == 0 || (post[0].op == HCAMD_MAP_IN && post[0].arg == 0));
  for (size_t i = 1; i < nPost && simple; ++i) {
    switch (post[i].op) {
    case HCAMD_MAP_ADDI: case HCAMD_MAP_SUBI: case HCAMD_MAP_MULI: case HCAMD_MAP_DIVI:
    case HCAMD_MAP_RSUBI: case HCAMD_MAP_RDIVI: case HCAMD_MAP_NEG: case HCAMD_MAP_ABS:
    case HCAMD_MAP_SQRT: case HCAMD_MAP_MSQRT: case HCAMD_MAP_MLOG:
      fp.op[fp.n] = post[i].op;
      fp.imm[fp.n++] = post[i].imm;
      break;
    case HCAMD_MAP_MDIVI: case HCAMD_MAP_RMDIVI: // (the fp16 flag of `arg`: an fp32 result has none)
      simple = (post[i].arg & 0x100u) == 0;
      fp.op[fp.n] = post[i].op;
      fp.imm[fp.n++] = post[i].imm;
      break;
    default:
      simple = false;
    }
  }
  if (simple) {
    Kernel *k = builtinKernel(dev, "map", "hcamd_cols_fold_f32");
    if (!k)
      return 1;
    const void *partial = workspace;
    size_t ld = colsPad;
    uint32_t nCols = static_cast<uint32_t>(cols), nBands = static_cast<uint32_t>(bands);
    void *args[] = {&partial, &ld, &out, &nCols, &nBands, &fp};
    const size_t grid[3] = {ceilDiv(cols, (size_t)256), 1, 1};
    const size_t block[3] = {1024, 1, 1};
    return launch(queue, k, grid, block, args, 0);
  }
  // the bands just written are the rows of an fp32 operand
  MapArgs a2{};
  ColArgs c2{};
  a2.in[0] = workspace;
  a2.ld[0] = colsPad;
  a2.rows = bands;
  a2.cols = cols;
  a2.n_instr = 1;
  a2.prog[0] = HcamdMapInstr{HCAMD_MAP_IN, 0, 0.0f};
  c2.kind = c.kind;
  c2.colsPad = c.colsPad;
  c2.band = static_cast<uint32_t>(bands);
  c2.lanes = static_cast<uint32_t>(colSecondLanes(bands, c.lanes));
  finishing(a2, c2);
  return launchOne(a2, c2, 1, 1);
}

namespace {
// Argument block of the row-program kernels (the same layout as in the device code).
struct RowStageDev {
  uint16_t begin, end;
  uint8_t kind, dst, loadMask;
  uint8_t masked;   // honour the inactive bits: numpy.ma's forms, or a row scalar read that may be deactivated
  uint16_t redMask; // row scalars this stage reads that may be deactivated
  uint8_t livePos;  // scalar stages: the result is active iff this row scalar is positive (0xff: not used)
  uint8_t frozen;   // STORE stages: deactivated elements are stored too, with what numpy.ma leaves in them
};
struct RowArgs {
  const void *in[kMapMaxIn];
  const void *col[kMapMaxIn];
  void *out;
  size_t ld[kMapMaxIn];
  size_t ldo;
  size_t rows, cols;
  uint32_t f16Mask, vecMask, interleaved;
  uint32_t nCol, nStages, passes;
  uint32_t hold, holdLast, allF32;
  RowStageDev stage[HCAMD_ROW_MAX_STAGES];
  HcamdMapInstr prog[HCAMD_ROW_MAX_INSTRS];
  uint8_t *deferred;   // chain kernels: one byte per row, 1 = left to the general kernel
  const uint8_t *only; // general kernel: the rows to run (null: all)
};

// A stage program that never holds two values at once, as the chain kernels
// take it: a push, then operations that change the value in place.  `x x mul`
// with two equal halves is such a program too, `x sq` (kRowSq exists between
// this file and the kernel only).  Appends to out[0 .. count) (never more
// instructions than it read); false: not a chain.
constexpr unsigned kRowSq = 63;
bool chainOf(const HcamdMapInstr *p, size_t n, HcamdMapInstr *out, size_t &count) {
  auto pushes = [](unsigned op) {
    return op == HCAMD_MAP_IN || op == HCAMD_MAP_CONST || op == HCAMD_MAP_RED;
  };
  auto inPlace = [](unsigned op) {
    return (op >= HCAMD_MAP_ADDI && op <= HCAMD_MAP_RDIV_IN) ||
           (op >= HCAMD_MAP_MDIVI && op <= HCAMD_MAP_MLOG) ||
           (op >= HCAMD_MAP_ADD_RED && op <= HCAMD_MAP_RMDIV_RED);
  };
  auto chain = [&](const HcamdMapInstr *q, size_t m) {
    if (m == 0 || !pushes(q[0].op))
      return false;
    for (size_t i = 1; i < m; ++i)
      if (!inPlace(q[i].op))
        return false;
    return true;
  };
  auto append = [&](const HcamdMapInstr *q, size_t m) {
    std::memcpy(out + count, q, m * sizeof(HcamdMapInstr));
    count += m;
  };
  if (chain(p, n)) {
    append(p, n);
    return true;
  }
  size_t k = 0;
  while (k < n && (pushes(p[k].op) || inPlace(p[k].op)))
    ++k;
  if (k == n || p[k].op != HCAMD_MAP_MUL || k < 2 || k % 2)
    return false;
  const size_t h = k / 2;
  if (!chain(p, h) || std::memcmp(p, p + h, h * sizeof(HcamdMapInstr)) != 0)
    return false;
  for (size_t i = k + 1; i < n; ++i)
    if (!inPlace(p[i].op))
      return false;
  append(p, h);
  const HcamdMapInstr sq{static_cast<uint16_t>(kRowSq), 0, 0.0f};
  append(&sq, 1);
  append(p + k + 1, n - k - 1);
  return true;
}
} // namespace

int hcamdLaunchRowProgram(OlQueue q, const HcamdMapInstr *prog,
                          const HcamdRowStage *stages, size_t nStages,
                          const void *const *inputs, const int *inputTypes,
                          const size_t *inputLd, size_t nInputs,
                          const void *const *columns, const int *columnTypes,
                          size_t nColumns, void *out, int outType, size_t ldo,
                          size_t rows, size_t cols) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *who = "hcamdLaunchRowProgram";
  auto typeOk = [](int t) { return t == HCAMD_F32 || t == HCAMD_F16; };
  if (!prog || !stages || nStages == 0 || nStages > HCAMD_ROW_MAX_STAGES) {
    dev->report("%s: %zu stages (1..%d allowed)", who, nStages, HCAMD_ROW_MAX_STAGES);
    return 1;
  }
  if (nInputs > kMapMaxIn || (nInputs && (!inputs || !inputTypes || !inputLd)) ||
      nColumns > kMapMaxIn || (nColumns && (!columns || !columnTypes))) {
    dev->report("%s: %zu operands and %zu columns (at most %zu each)", who, nInputs,
                nColumns, kMapMaxIn);
    return 1;
  }
  if (!typeOk(outType)) {
    dev->report("%s: unsupported output type %d", who, outType);
    return 1;
  }
  RowArgs a{};
  // Every stage must keep the stack within bounds, leave one value, and read
  // only operands that exist and row scalars that have been written.  Along
  // the way: which row scalars the data can deactivate (a fold over elements
  // that numpy.ma's forms can deactivate, a scalar stage with such a form, and
  // everything computed from one of those), and which stages read them.
  uint32_t written = (1u << nColumns) - 1u;
  uint32_t deadable = 0;
  bool tracking = false; // some row scalar may be deactivated, or active elements are counted
  // ... for a reason other than an operation on row scalars that can fail (a
  // quotient, a root, a logarithm): counted folds, folds over elements that can be
  // deactivated, frozen stores, per-row results that are tiles
  bool trackingBeyondScalars = false;
  uint32_t usedIn[HCAMD_ROW_MAX_STAGES] = {};
  size_t pc = 0;
  for (size_t s = 0; s < nStages; ++s) {
    const HcamdRowStage &st = stages[s];
    if (st.kind > HCAMD_ROW_COUNT || st.nInstr == 0 ||
        pc + st.nInstr > HCAMD_ROW_MAX_INSTRS) {
      dev->report("%s: stage %zu: kind %u with %u instructions (%d in all allowed)", who,
                  s, st.kind, st.nInstr, HCAMD_ROW_MAX_INSTRS);
      return 1;
    }
    const bool stores = st.kind == HCAMD_ROW_STORE || st.kind == HCAMD_ROW_STORE_COL;
    if (stores != (s + 1 == nStages)) {
      dev->report("%s: the last stage, and only the last, must store", who);
      return 1;
    }
    const bool perElement = !(st.kind == HCAMD_ROW_SCALAR || st.kind == HCAMD_ROW_STORE_COL);
    if (!stores && st.dst >= HCAMD_ROW_MAX_SCALARS) {
      dev->report("%s: stage %zu writes row scalar %u (%d exist)", who, s, st.dst,
                  HCAMD_ROW_MAX_SCALARS);
      return 1;
    }
    int sp = 0;
    bool hasForms = false;
    uint32_t readsDeadable = 0;
    a.stage[s].livePos = 0xff;
    size_t stageEnd = pc + st.nInstr;
    if (prog[stageEnd - 1].op == HCAMD_MAP_LIVEPOS) {
      const unsigned index = prog[stageEnd - 1].arg & 0xffu;
      if (perElement || st.nInstr < 2 || index >= HCAMD_ROW_MAX_SCALARS || !((written >> index) & 1)) {
        dev->report("%s: stage %zu: LIVEPOS closes a scalar stage and names a row scalar that "
                    "has been written", who, s);
        return 1;
      }
      a.stage[s].livePos = static_cast<uint8_t>(index);
      --stageEnd;
    }
    bool frozen = false;
    if (prog[stageEnd - 1].op == HCAMD_MAP_FROZEN) {
      if (st.kind != HCAMD_ROW_STORE || st.nInstr < 2) {
        dev->report("%s: stage %zu: FROZEN closes a STORE stage", who, s);
        return 1;
      }
      frozen = true;
      a.stage[s].frozen = 1;
      --stageEnd;
    }
    for (size_t i = pc; i < stageEnd; ++i) {
      const unsigned op = prog[i].op;
      int pops, pushes;
      const bool maskedRed = op == HCAMD_MAP_MDIV_RED || op == HCAMD_MAP_RMDIV_RED;
      if ((op >= HCAMD_MAP_MDIV && op <= HCAMD_MAP_MLOG && op != HCAMD_MAP_CLEAR) || maskedRed ||
          op == HCAMD_MAP_MASQRT)
        hasForms = true;
      const bool red = op >= HCAMD_MAP_RED && op <= HCAMD_MAP_RED0;
      if (red)
        pops = (op == HCAMD_MAP_RED || op == HCAMD_MAP_RED0) ? 0 : 1, pushes = 1;
      else if (op == HCAMD_MAP_MASQRT && !perElement)
        pops = 1, pushes = 1;
      else
        mapStackEffectMasked(op, pops, pushes);
      if (pops < 0) {
        dev->report("%s: unknown opcode %u at %zu", who, op, i);
        return 1;
      }
      const bool maskedIn = op == HCAMD_MAP_MDIV_IN || op == HCAMD_MAP_RMDIV_IN;
      const bool readsOperand = op == HCAMD_MAP_IN || maskedIn ||
                                (op >= HCAMD_MAP_ADD_IN && op <= HCAMD_MAP_RDIV_IN);
      // (bits 8 and up of `arg` are flags: fp16, and in scalar stages the form of the operation)
      const unsigned index = (maskedIn || red || frozen) ? prog[i].arg & 0xffu : prog[i].arg;
      if (readsOperand) {
        if (!perElement || index >= nInputs) {
          dev->report("%s: operand %u at %zu (%zu given; scalar stages read none)", who,
                      index, i, nInputs);
          return 1;
        }
        usedIn[s] |= 1u << index;
      }
      if (op == HCAMD_MAP_RED0 && perElement) {
        dev->report("%s: opcode %u at %zu outside a scalar stage", who, op, i);
        return 1;
      }
      if (perElement && !frozen && !red && !maskedIn && (prog[i].arg & ~0x1ffu)) {
        dev->report("%s: flags 0x%x at %zu outside a scalar or frozen stage", who, prog[i].arg, i);
        return 1;
      }
      if (red && (index >= HCAMD_ROW_MAX_SCALARS || !((written >> index) & 1))) {
        dev->report("%s: row scalar %u read at %zu before it is written", who, index, i);
        return 1;
      }
      if (red && op != HCAMD_MAP_RED0)
        readsDeadable |= (1u << index) & deadable;
      // CLEAR makes every element active again: a deactivated row scalar read
      // before it (the operand of a NumPy function, computed on its value) does
      // not take the row out of the store
      if (op == HCAMD_MAP_CLEAR && perElement)
        readsDeadable = 0;
      if (sp < pops) {
        dev->report("%s: stack underflow at %zu", who, i);
        return 1;
      }
      sp += pushes - pops;
      if (sp > (frozen ? 1 : kMapDepth)) {
        dev->report("%s: stack deeper than %d at %zu", who, frozen ? 1 : kMapDepth, i);
        return 1;
      }
    }
    if (sp != 1) {
      dev->report("%s: stage %zu leaves %d values, expected 1", who, s, sp);
      return 1;
    }
    a.stage[s].begin = static_cast<uint16_t>(pc);
    a.stage[s].end = static_cast<uint16_t>(stageEnd);
    a.stage[s].kind = static_cast<uint8_t>(st.kind);
    a.stage[s].dst = static_cast<uint8_t>(st.dst);
    a.stage[s].redMask = static_cast<uint16_t>(readsDeadable);
    a.stage[s].masked = (hasForms || readsDeadable || frozen) ? 1 : 0;
    const bool canDie = (stores || st.kind == HCAMD_ROW_COUNT) ? false
                        : perElement                           ? (hasForms || readsDeadable)
                                                   : (hasForms || readsDeadable || a.stage[s].livePos != 0xff);
    if (!stores) {
      written |= 1u << st.dst;
      deadable = canDie ? deadable | (1u << st.dst) : deadable & ~(1u << st.dst);
    }
    // (a STORE_COL stage that can fail stores what numpy.ma leaves: the scalar interpreter's business too)
    tracking = tracking || canDie || frozen || st.kind == HCAMD_ROW_COUNT ||
               (st.kind == HCAMD_ROW_STORE_COL && st.dst != 0) ||
               (!perElement && (hasForms || readsDeadable));
    trackingBeyondScalars = trackingBeyondScalars || frozen || st.kind == HCAMD_ROW_COUNT ||
                            (st.kind == HCAMD_ROW_STORE_COL && st.dst != 0) ||
                            (perElement && !stores && hasForms) || a.stage[s].livePos != 0xff;
    pc += st.nInstr;
  }
  std::memcpy(a.prog, prog, pc * sizeof(HcamdMapInstr));
  if (rows == 0 || cols == 0)
    return 0;
  if (!out) {
    dev->report("%s: null pointer", who);
    return 1;
  }
  const bool storesTile = stages[nStages - 1].kind == HCAMD_ROW_STORE;
  if (storesTile && rows > 1 && ldo < cols) {
    dev->report("%s: leading dimension smaller than cols", who);
    return 1;
  }
  if (cols >= ((size_t)1 << 32) || rows > ((size_t)1 << 31)) {
    dev->report("%s: more than 2^31 rows or 2^32 - 1 columns", who);
    return 1;
  }
  char name[48];
  const size_t perRow = cols / 8 + (cols % 8 ? 1 : 0);
  // a wave per row up to 4096 columns (at most 8 chunks per lane), else a workgroup
  const size_t lanesPerRow = perRow <= 512 ? 64 : 256;
  const size_t passes = ceilDiv(perRow, lanesPerRow);
  for (size_t i = 0; i < nInputs; ++i) {
    if (!inputs[i]) {
      dev->report("%s: null pointer", who);
      return 1;
    }
    if (!typeOk(inputTypes[i])) {
      dev->report("%s: unsupported operand type %d", who, inputTypes[i]);
      return 1;
    }
    if (inputLd[i] != 0 && rows > 1 && inputLd[i] < cols) {
      dev->report("%s: leading dimension smaller than cols", who);
      return 1;
    }
    const size_t esz = inputTypes[i] == HCAMD_F16 ? 2 : 4;
    a.in[i] = inputs[i];
    a.ld[i] = inputLd[i];
    if (inputTypes[i] == HCAMD_F16)
      a.f16Mask |= 1u << i;
    if (cols >= 8 && aligned16(inputs[i]) && (rows == 1 || (inputLd[i] * esz) % 16 == 0))
      a.vecMask |= 1u << i;
  }
  for (size_t k = 0; k < nColumns; ++k) {
    if (!columns[k] || !typeOk(columnTypes[k])) {
      dev->report("%s: column %zu: null pointer or unsupported type", who, k);
      return 1;
    }
    a.col[k] = columns[k];
    if (columnTypes[k] == HCAMD_F16)
      a.f16Mask |= 1u << (16 + k);
  }
  if (outType == HCAMD_F16)
    a.f16Mask |= 1u << 8;
  if (storesTile && cols >= 8 && aligned16(out) &&
      (rows == 1 || (ldo * (outType == HCAMD_F16 ? 2 : 4)) % 16 == 0))
    a.vecMask |= 1u << 8;
  a.out = out;
  a.ldo = ldo;
  a.rows = rows;
  a.cols = cols;
  a.nCol = static_cast<uint32_t>(nColumns);
  a.nStages = static_cast<uint32_t>(nStages);
  a.passes = static_cast<uint32_t>(passes);
  uint32_t used = 0;
  for (size_t s = 0; s < nStages; ++s) {
    a.stage[s].loadMask = static_cast<uint8_t>(usedIn[s]);
    used |= usedIn[s];
  }
  // 16-byte accesses need every operand in use and a stored tile to allow them;
  // otherwise the columns are dealt to the lanes one by one and every access
  // is element-wise but coalesced.
  if ((used & ~a.vecMask & 0xffu) || (storesTile && !((a.vecMask >> 8) & 1))) {
    a.vecMask = 0;
    a.interleaved = 1;
  }
  // A layer normalisation as the front-end emits it for a body written with
  // mean and var along axis 1 (six stages: the mean, the centred squares, the
  // variance, the scale, then (x - mean) / s * w + b; the mean's division and the
  // last one numpy.ma's), on dense fp32 rows of at most 32768 elements with
  // fp32 vectors w and b: a kernel that interprets nothing, and stores nothing
  // to a row whose mean is not finite, as the stages demand (variant 2 of
  // "rows": the general kernel for this too; variant 1: for everything).
  {
    auto is = [&](size_t at, unsigned op, unsigned arg) {
      return prog[at].op == op && prog[at].arg == arg;
    };
    auto launchNorm = [&](bool rmsForm, const void *x, size_t ldx, const void *w, const void *b,
                          float n, float eps, bool half = false, uint32_t frozen = 0) {
      const size_t chunks = cols / (half ? 8 : 4);
      // two chunks to a lane on up to 512 lanes, then four; 1024 lanes from 2048 chunks on
      size_t lpr = 64, e = chunks <= 64 ? 1 : 2;
      while (lpr < 512 && lpr * 2 < chunks)
        lpr *= 2;
      if (chunks > 2048)
        lpr = 1024;
      while (lpr * e < chunks)
        e *= 2;
      // variants of "norm", for measurements: 1 twice the lanes to a row, 2 half of them
      if (variantOf("norm") == 1 && lpr < 1024 && e > 1)
        lpr *= 2, e /= 2;
      else if (variantOf("norm") == 2 && lpr > 64 && e < 8)
        lpr /= 2, e *= 2;
      std::snprintf(name, sizeof name, "hcamd_%s_norm_%s_w%zu_e%zu", rmsForm ? "rms" : "layer",
                    half ? "f16" : "f32", lpr, e);
      const size_t t = std::max(lpr, (size_t)256);
      size_t ldOut = ldo;
      uint32_t nRows = static_cast<uint32_t>(rows), nCols = static_cast<uint32_t>(cols);
      void *args[] = {&x, &ldx, &w, &b, &out, &ldOut, &nRows, &nCols, &n, &eps, &frozen};
      return launch1d(queue, "map", name, ceilDiv(rows, t / lpr), t, args);
    };
    auto stage = [&](size_t s, unsigned kind, unsigned dst, unsigned n) {
      return stages[s].kind == kind && (kind == HCAMD_ROW_STORE || stages[s].dst == dst) &&
             stages[s].nInstr == n;
    };
    const bool shape =
        variantOf("rows") == 0 && nStages == 6 && nInputs == 3 && nColumns == 0 && pc == 18 &&
        stage(0, HCAMD_ROW_SUM, 0, 1) && stage(1, HCAMD_ROW_SCALAR, 1, 2) &&
        stage(2, HCAMD_ROW_SUM, 2, 5) && stage(3, HCAMD_ROW_SCALAR, 3, 2) &&
        stage(4, HCAMD_ROW_SCALAR, 4, 3) && stage(5, HCAMD_ROW_STORE, 0, 5);
    if (shape && is(0, HCAMD_MAP_IN, 0) && is(1, HCAMD_MAP_RED, 0) && is(2, HCAMD_MAP_MDIVI, 0) &&
        is(3, HCAMD_MAP_IN, 0) && is(4, HCAMD_MAP_SUB_RED, 1) && is(5, HCAMD_MAP_IN, 0) &&
        is(6, HCAMD_MAP_SUB_RED, 1) && is(7, HCAMD_MAP_MUL, 0) && is(8, HCAMD_MAP_RED0, 2) &&
        is(9, HCAMD_MAP_DIVI, 0) && is(10, HCAMD_MAP_RED, 3) && is(11, HCAMD_MAP_ADDI, 0) &&
        is(12, HCAMD_MAP_MSQRT, 0) && is(13, HCAMD_MAP_IN, 0) && is(14, HCAMD_MAP_SUB_RED, 1) &&
        is(15, HCAMD_MAP_MDIV_RED, 4) && is(16, HCAMD_MAP_MUL_IN, 1) &&
        is(17, HCAMD_MAP_ADD_IN, 2) && prog[2].imm == prog[9].imm && prog[11].imm >= 0.0f &&
        a.f16Mask == 0 &&
        inputLd[0] != 0 && inputLd[1] == 0 && inputLd[2] == 0 && (a.vecMask & 0x107u) == 0x107u &&
        cols % 4 == 0 && cols <= 32768) {
      return launchNorm(false, inputs[0], inputLd[0], inputs[1], inputs[2], prog[2].imm, prog[11].imm);
    }
    // The root-mean-square normalisation  x / sqrt(mean(x * x) + eps) * w  in its
    // three stages, under the same conditions (a row whose mean of squares is not
    // finite is left alone).
    const bool rms =
        variantOf("rows") == 0 && nStages == 3 && nInputs == 2 && nColumns == 0 && pc == 9 &&
        stage(0, HCAMD_ROW_SUM, 0, 2) && stage(1, HCAMD_ROW_SCALAR, 1, 4) &&
        stage(2, HCAMD_ROW_STORE, 0, 3);
    const bool rmsScale = is(2, HCAMD_MAP_RED, 0) && is(3, HCAMD_MAP_MDIVI, 0) &&
                          is(4, HCAMD_MAP_ADDI, 0) && is(5, HCAMD_MAP_MSQRT, 0) &&
                          prog[4].imm >= 0.0f;
    if (rms && is(0, HCAMD_MAP_IN, 0) && is(1, HCAMD_MAP_MUL_IN, 0) && rmsScale &&
        is(6, HCAMD_MAP_IN, 0) && is(7, HCAMD_MAP_MDIV_RED, 1) && is(8, HCAMD_MAP_MUL_IN, 1) &&
        a.f16Mask == 0 && inputLd[0] != 0 && inputLd[1] == 0 && (a.vecMask & 0x103u) == 0x103u &&
        cols % 4 == 0 && cols <= 32768)
      return launchNorm(true, inputs[0], inputLd[0], inputs[1], inputs[1], prog[3].imm, prog[4].imm);
    // The same on fp16 rows, computed in fp32 and stored as fp16 (the program
    // then ends in R16); w stays fp32.
    // (with FROZEN at the end when the body computes from x.astype(float32), a
    // bare numpy.ma array: every element is stored, a deactivated one as x)
    const bool rmsFrozen = pc == 11 && prog[10].op == HCAMD_MAP_FROZEN;
    const bool rmsHalf =
        variantOf("rows") == 0 && nStages == 3 && nInputs == 2 && nColumns == 0 &&
        (pc == 10 || rmsFrozen) && stage(0, HCAMD_ROW_SUM, 0, 2) && stage(1, HCAMD_ROW_SCALAR, 1, 4) &&
        stage(2, HCAMD_ROW_STORE, 0, rmsFrozen ? 5 : 4);
    if (rmsHalf && is(0, HCAMD_MAP_IN, 0) && is(1, HCAMD_MAP_MUL_IN, 0) && rmsScale &&
        is(6, HCAMD_MAP_IN, 0) && is(7, HCAMD_MAP_MDIV_RED, 1) && is(8, HCAMD_MAP_MUL_IN, 1) &&
        is(9, HCAMD_MAP_R16, 0) && a.f16Mask == 0x101u && inputLd[0] != 0 && inputLd[1] == 0 &&
        (a.vecMask & 0x103u) == 0x103u && cols % 8 == 0 && cols <= 65536)
      return launchNorm(true, inputs[0], inputLd[0], inputs[1], inputs[1], prog[3].imm, prog[4].imm,
                        true, rmsFrozen ? 1u : 0u);
  }
  // Rows of whole, aligned chunks, at most 4096 of them, whose stages are all
  // chains run on the chain kernels: a lane has its whole part of the row at
  // once, 8, 16 or 32 elements to a dispatch, and the operand that most
  // instructions read stays in LDS for the row (variant 1 of "rows": never).
  size_t lanes = lanesPerRow, maxGroups = SIZE_MAX, threads = 256;
  std::snprintf(name, sizeof name, "hcamd_row_program_w%zu", lanes);
  // A program whose only deactivations are failed operations on row scalars
  // takes two launches: the chain kernel for every row, which leaves a row alone
  // and marks it when such an operation fails on it, then the general kernel for
  // the marked rows (variant 3 of "rows": the general kernel alone, as for
  // every other program that needs the books).
  const bool twoLaunches = tracking && !trackingBeyondScalars && variantOf("rows") == 0;
  RowArgs general = a;
  char generalName[64];
  std::snprintf(generalName, sizeof generalName, "%s", name);
  const size_t generalLanes = lanes;
  bool chainTaken = false;
  if (variantOf("rows") != 1 && (!tracking || twoLaunches) && !a.interleaved && cols % 8 == 0 && perRow <= 4096 &&
      nInputs > 0) {
    HcamdMapInstr chained[HCAMD_ROW_MAX_INSTRS];
    size_t nChained = 0;
    uint16_t begin[HCAMD_ROW_MAX_STAGES], end[HCAMD_ROW_MAX_STAGES];
    bool ok = true;
    size_t at = 0;
    for (size_t s = 0; s < nStages && ok; ++s) {
      begin[s] = static_cast<uint16_t>(nChained);
      ok = chainOf(prog + at, stages[s].nInstr, chained, nChained);
      end[s] = static_cast<uint16_t>(nChained);
      at += stages[s].nInstr;
    }
    uint32_t reads[kMapMaxIn] = {};
    for (size_t i = 0; i < nChained; ++i) {
      const HcamdMapInstr &in = chained[i];
      const unsigned op = in.op;
      if (op == HCAMD_MAP_IN || (op >= HCAMD_MAP_ADD_IN && op <= HCAMD_MAP_RDIV_IN) ||
          op == HCAMD_MAP_MDIV_IN || op == HCAMD_MAP_RMDIV_IN)
        ++reads[in.arg & 3u];
    }
    size_t hold = 0;
    for (size_t i = 1; i < nInputs; ++i)
      if (reads[i] > reads[hold])
        hold = i;
    if (ok && reads[hold] > 0) {
      // one, two or four chunks per lane of a wave, then four on more lanes
      const unsigned p = perRow <= 64 ? 1 : perRow <= 128 ? 2 : 4;
      lanes = 64;
      while (lanes * p < perRow)
        lanes *= 2;
      threads = std::max<size_t>(256, lanes);
      for (size_t s = 0; s < nStages; ++s) {
        a.stage[s].begin = begin[s];
        a.stage[s].end = end[s];
      }
      std::memset(a.prog, 0, sizeof a.prog);
      std::memcpy(a.prog, chained, nChained * sizeof(HcamdMapInstr));
      a.hold = static_cast<uint32_t>(hold);
      // storesTile: the output is a tile; a per-row result has no layout to agree with
      a.allF32 = (a.f16Mask & used & 0xffu) == 0 && (!storesTile || outType == HCAMD_F32) ? 1u : 0u;
      for (size_t i = 0; i < nChained; ++i) {
        const unsigned op = chained[i].op;
        if ((op == HCAMD_MAP_IN || (op >= HCAMD_MAP_ADD_IN && op <= HCAMD_MAP_RDIV_IN) ||
             op == HCAMD_MAP_MDIV_IN || op == HCAMD_MAP_RMDIV_IN) &&
            (chained[i].arg & 3u) == hold)
          a.holdLast = static_cast<uint32_t>(i);
      }
      std::snprintf(name, sizeof name, "hcamd_row_program_chain_w%zu_p%u", lanes, p);
      // these kernels walk the rows themselves: as many workgroups as are resident at once
      maxGroups = (size_t)computeUnitsOf(dev) * (p <= 2 ? 24 : 16) / (threads / 64); // 6 or 4 waves per SIMD
      chainTaken = true;
    }
  }
  if (tracking && !chainTaken) // (the rewrite above is for the chain kernels only)
    a = general;
  if (tracking && chainTaken) {
    // one byte per row, kept with the device and grown when a launch has more rows
    if (dev->rowMarksBytes < rows) {
      if (dev->rowMarks)
        (void)hipFree(dev->rowMarks);
      dev->rowMarks = nullptr;
      dev->rowMarksBytes = 0;
      const size_t want = std::max(rows, (size_t)1 << 16);
      if (hipMalloc(&dev->rowMarks, want) != hipSuccess) {
        dev->report("%s: no device memory for %zu row marks", who, want);
        return 1;
      }
      dev->rowMarksBytes = want;
    }
    a.deferred = static_cast<uint8_t *>(dev->rowMarks);
    general.only = static_cast<const uint8_t *>(dev->rowMarks);
  }
  Kernel *k = builtinKernel(dev, "map", name);
  if (!k)
    return 1;
  void *args[] = {&a};
  const size_t grid[3] = {std::min(ceilDiv(rows, threads / lanes), maxGroups), 1, 1};
  const size_t block[3] = {threads, 1, 1};
  if (int rc = launch(queue, k, grid, block, args, 0))
    return rc;
  if (!(tracking && chainTaken))
    return 0;
  Kernel *kg = builtinKernel(dev, "map", generalName);
  if (!kg)
    return 1;
  void *gargs[] = {&general};
  const size_t ggrid[3] = {ceilDiv(rows, (size_t)256 / generalLanes), 1, 1};
  const size_t gblock[3] = {256, 1, 1};
  return launch(queue, kg, ggrid, gblock, gargs, 0);
}

int hcamdLaunchPairwiseDistF32(OlQueue q, const float *a, size_t lda,
                               const float *b, size_t ldb, float *out,
                               size_t ldo, size_t m, size_t n,
                               size_t d) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  if (m == 0 || n == 0)
    return 0;
  if (!a || !b || !out) {
    dev->report("hcamdLaunchPairwiseDistF32: null pointer");
    return 1;
  }
  if ((m > 1 && lda < d) || (n > 1 && ldb < d) || (m > 1 && ldo < n)) {
    dev->report("hcamdLaunchPairwiseDistF32: leading dimension smaller than the row");
    return 1;
  }
  const size_t gy = ceilDiv(m, 64);
  if (gy > 65535) {
    dev->report("hcamdLaunchPairwiseDistF32: more than 65535 x 64 rows");
    return 1;
  }
  Kernel *k = builtinKernel(dev, "distance", "hcamd_pairwise_dist_f32");
  if (!k)
    return 1;
  void *args[] = {&a, &lda, &b, &ldb, &out, &ldo, &m, &n, &d};
  const size_t grid[3] = {ceilDiv(n, 64), gy, 1};
  const size_t block[3] = {256, 1, 1};
  return launch(queue, k, grid, block, args, 0);
}

// ---------------------------------------------------------------------------
// Matrix product of gathered tiles
// ---------------------------------------------------------------------------
struct HcamdGatherGemm_ {
  Device *device = nullptr;
  int32_t *tables = nullptr; // one device allocation holding all seven tables
  size_t offGroups = 0, offRows[3] = {0, 0, 0}, offCols[3] = {0, 0, 0};
  size_t elems[3] = {0, 0, 0}; // span of each buffer in elements
  uint32_t tm = 0, tn = 0, k = 0, nGroups = 0;
  uint32_t fuse = 1, nSets = 0; // records per workgroup, number of workgroups
  // distinct b windows, their table, and the scratch their packed tiles live in
  uint32_t nWindows = 0, kPad = 0, tnPad = 0;
  size_t offWindows = 0;
  float *bpack = nullptr;
};

namespace {
// must match GatherGemmArgs and PackBArgs in kernels/gather.hip
struct GatherGemmArgs {
  const void *a;
  const float *bpack;
  void *out;
  const int32_t *groups;
  const int32_t *a_rows, *a_cols, *o_rows, *o_cols;
  uint32_t tm, tn, k, n_groups, per_xcd;
  uint32_t k_pad, tn_pad;
};
struct PackBArgs {
  const void *b;
  float *bpack;
  const int32_t *windows;
  const int32_t *b_rows, *b_cols;
  uint32_t k, tn, k_pad, tn_pad, n_windows;
};

constexpr int kGatherEntry = 8;   // ints per row / column entry
constexpr int kGatherRecord = 16; // ints per group record

// Fills the entries of one tile axis of one operand.  `mine` says which
// dimensions this axis drives (the others contribute index 0).
void gatherEntries(const HcamdGatherOperand &op, const int32_t *index, size_t n,
                   const bool mine[4], int32_t *dst) {
  for (size_t r = 0; r < n; ++r) {
    int32_t *e = dst + r * kGatherEntry;
    int64_t off = 0;
    bool inside = true;
    for (int d = 0; d < 4; ++d) {
      int32_t idx = 0;
      if (d < op.ndim && mine[d])
        idx = index[r * op.ndim + d];
      e[1 + d] = idx;
      const int64_t size = d < op.ndim ? (int64_t)op.shape[d] : 1;
      if (idx < 0 || idx >= size)
        inside = false;
      else if (d < op.ndim)
        off += (int64_t)idx * (int64_t)op.strides[d];
    }
    e[0] = inside ? (int32_t)off : 0; // never used when some index is outside
    e[5] = e[6] = e[7] = 0;
  }
}
} // namespace

HcamdGatherGemm hcamdGatherGemmCreate(OlQueue q, const HcamdGatherOperand *a,
                                      const HcamdGatherOperand *b,
                                      const HcamdGatherOperand *out,
                                      size_t nGroups, size_t tm, size_t tn,
                                      size_t k) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return nullptr;
  Device *dev = queue->device;
  if (!a || !b || !out) {
    dev->report("hcamdGatherGemmCreate: null operand");
    return nullptr;
  }
  if (nGroups == 0 || tm == 0 || tn == 0 || nGroups > 0x7ffffff0ull ||
      tm > 0x7fffffffull || tn > 0x7fffffffull || k > 0x7fffffffull) {
    dev->report("hcamdGatherGemmCreate: invalid sizes (groups %zu, tile %zu x "
                "%zu x %zu)", nGroups, tm, tn, k);
    return nullptr;
  }
  const HcamdGatherOperand *ops[3] = {a, b, out};
  const size_t rows[3] = {tm, k, tm}, cols[3] = {k, tn, tn};
  static const char *const names[3] = {"a", "b", "out"};
  bool rowDim[3][4], colDim[3][4];
  size_t span[3];
  for (int o = 0; o < 3; ++o) {
    const HcamdGatherOperand &op = *ops[o];
    if (op.ndim < 1 || op.ndim > 4 || !op.starts ||
        (rows[o] && !op.rowIndex) || (cols[o] && !op.colIndex)) {
      dev->report("hcamdGatherGemmCreate: operand %s: rank %d or null table",
                  names[o], op.ndim);
      return nullptr;
    }
    size_t last = 0;
    for (int d = 0; d < op.ndim; ++d) {
      if (op.shape[d] == 0) {
        dev->report("hcamdGatherGemmCreate: operand %s is empty", names[o]);
        return nullptr;
      }
      last += (op.shape[d] - 1) * op.strides[d];
    }
    if (last >= 0x7fffffffull) {
      dev->report("hcamdGatherGemmCreate: operand %s spans more than 2^31 "
                  "elements", names[o]);
      return nullptr;
    }
    span[o] = last + 1;
    for (int d = 0; d < 4; ++d) {
      bool r = false, c = false;
      if (d < op.ndim) {
        for (size_t i = 0; i < rows[o] && !r; ++i)
          r = op.rowIndex[i * op.ndim + d] != 0;
        for (size_t i = 0; i < cols[o] && !c; ++i)
          c = op.colIndex[i * op.ndim + d] != 0;
      }
      if (r && c) {
        dev->report("hcamdGatherGemmCreate: operand %s: dimension %d depends on "
                    "both tile coordinates", names[o], d);
        return nullptr;
      }
      colDim[o][d] = c;
      rowDim[o][d] = !c; // constants (all-zero tables) ride with the row
    }
    for (size_t g = 0; g < nGroups; ++g)
      for (int d = 0; d < op.ndim; ++d)
        if (op.starts[g * op.ndim + d] < 0) {
          dev->report("hcamdGatherGemmCreate: operand %s: negative window start",
                      names[o]);
          return nullptr;
        }
  }

  // Groups may run in any order.  They are laid out by the address of their
  // windows, so that workgroups that are resident together, and the run of
  // groups each XCD receives, touch neighbouring memory: windows that overlap or
  // share cache lines are then served by one L2 fill.  Sorted by (b, a), runs
  // of records that read the same b window can be fused, G to a workgroup
  // (kernels/gather.hip); unfused, the order is (a, b).
  std::vector<uint32_t> order;
  std::vector<int64_t> key;
  try {
    order.resize(nGroups);
    key.assign(nGroups * 2, 0);
  } catch (...) {
    dev->report("hcamdGatherGemmCreate: out of host memory");
    return nullptr;
  }
  for (size_t g = 0; g < nGroups; ++g) {
    order[g] = (uint32_t)g;
    for (int o = 0; o < 2; ++o) {
      const HcamdGatherOperand &op = *ops[o];
      for (int d = 0; d < op.ndim; ++d)
        key[g * 2 + o] += (int64_t)op.starts[g * op.ndim + d] * (int64_t)op.strides[d];
    }
  }
  auto sortBy = [&](int first) {
    std::stable_sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) {
      const int64_t x0 = key[2 * (size_t)x + first], y0 = key[2 * (size_t)y + first];
      if (x0 != y0)
        return x0 < y0;
      return key[2 * (size_t)x + 1 - first] < key[2 * (size_t)y + 1 - first];
    });
  };
  sortBy(1);
  auto sameB = [&](size_t x, size_t y) {
    for (int d = 0; d < b->ndim; ++d)
      if (b->starts[x * b->ndim + d] != b->starts[y * b->ndim + d])
        return false;
    return true;
  };
  // G = 4 needs the 64-row block; small tiles fuse in pairs.  Fusion must leave
  // enough workgroups to fill the device.  A run of records with one b window
  // is padded with empty records (extent 0) to a multiple of G, so that no set
  // mixes two b windows.
  const int wanted = variantOf("gather_fuse");
  const size_t cus = (size_t)std::max(computeUnitsOf(dev), 1);
  size_t fuse = wanted >= 16 ? 16 : wanted >= 4 ? 4 : wanted >= 2 ? 2 : 1;
  if (wanted == 0) {
    // workgroups a launch would have with G records fused (64-row blocks)
    auto groupsOf = [&](size_t G) {
      return nGroups / G * ceilDiv(G * tm, (size_t)64) * ceilDiv(tn, (size_t)64);
    };
    // (16 records per workgroup measured slower than 4 on the shapes tried:
    // more registers, fewer resident waves; it stays selectable)
    if (tm >= 16 && groupsOf(4) >= cus)
      fuse = 4;
    else if (nGroups / 2 >= cus)
      fuse = 2;
  }
  std::vector<int64_t> slots; // record in each slot, -1 = empty
  try {
    slots.reserve(nGroups + fuse);
    if (fuse == 1) {
      sortBy(0);
      for (size_t i = 0; i < nGroups; ++i)
        slots.push_back(order[i]);
    } else {
      for (size_t i = 0; i < nGroups; ++i) {
        if (i > 0 && !sameB(order[i - 1], order[i]))
          while (slots.size() % fuse)
            slots.push_back(-1);
        slots.push_back(order[i]);
      }
      while (slots.size() % fuse)
        slots.push_back(-1);
    }
  } catch (...) {
    dev->report("hcamdGatherGemmCreate: out of host memory");
    return nullptr;
  }
  const size_t nSets = slots.size() / fuse;
  if (nSets > 0x7ffffff0ull) {
    dev->report("hcamdGatherGemmCreate: too many groups");
    return nullptr;
  }

  auto plan = new (std::nothrow) HcamdGatherGemm_;
  if (!plan)
    return nullptr;
  plan->device = dev;
  plan->tm = (uint32_t)tm;
  plan->tn = (uint32_t)tn;
  plan->k = (uint32_t)k;
  plan->nGroups = (uint32_t)nGroups;
  plan->fuse = (uint32_t)fuse;
  plan->nSets = (uint32_t)nSets;
  // distinct b windows in slot order: index per group, representative group
  std::vector<uint32_t> windowOf, windowRep;
  try {
    windowOf.assign(nGroups, 0);
    std::vector<uint32_t> byB(order); // groups with equal b windows adjacent
    std::stable_sort(byB.begin(), byB.end(), [&](uint32_t x, uint32_t y) {
      for (int d = 0; d < b->ndim; ++d) {
        const int32_t sx = b->starts[(size_t)x * b->ndim + d],
                      sy = b->starts[(size_t)y * b->ndim + d];
        if (sx != sy)
          return sx < sy;
      }
      return false;
    });
    for (size_t i = 0; i < nGroups; ++i) {
      if (i == 0 || !sameB(byB[i - 1], byB[i]))
        windowRep.push_back(byB[i]);
      windowOf[byB[i]] = (uint32_t)windowRep.size() - 1;
    }
  } catch (...) {
    dev->report("hcamdGatherGemmCreate: out of host memory");
    delete plan;
    return nullptr;
  }
  plan->nWindows = (uint32_t)windowRep.size();
  plan->kPad = (uint32_t)(ceilDiv(k, 32) * 32);
  plan->tnPad = (uint32_t)(ceilDiv(tn, 4) * 4);
  if (windowRep.size() > 65535) {
    dev->report("hcamdGatherGemmCreate: more than 65535 distinct b windows");
    delete plan;
    return nullptr;
  }
  size_t total = 0;
  plan->offGroups = total;
  total += nSets * fuse * kGatherRecord; // records past nGroups stay empty (extent 0)
  plan->offWindows = total;
  total += windowRep.size() * 8;
  for (int o = 0; o < 3; ++o) {
    plan->elems[o] = span[o];
    plan->offRows[o] = total;
    total += rows[o] * kGatherEntry;
    plan->offCols[o] = total;
    total += cols[o] * kGatherEntry;
  }
  total += 4; // keeps the allocation non-empty and the last entry padded
  std::vector<int32_t> host;
  try {
    host.assign(total, 0);
  } catch (...) {
    dev->report("hcamdGatherGemmCreate: out of host memory");
    delete plan;
    return nullptr;
  }
  for (size_t slot = 0; slot < slots.size(); ++slot) {
    if (slots[slot] < 0)
      continue; // stays all zero: nothing is inside an empty window
    const size_t g = (size_t)slots[slot];
    int32_t *rec = host.data() + plan->offGroups + slot * kGatherRecord;
    for (int o = 0; o < 3; ++o) {
      const HcamdGatherOperand &op = *ops[o];
      int32_t *w = rec + 5 * o;
      int64_t base = 0;
      bool empty = false;
      for (int d = 0; d < 4; ++d) {
        int64_t ext = 1;
        if (d < op.ndim) {
          const int64_t st = op.starts[g * op.ndim + d];
          ext = (int64_t)op.shape[d] - st;
          base += st * (int64_t)op.strides[d];
        }
        if (ext <= 0) {
          ext = 0;
          empty = true;
        }
        w[1 + d] = (int32_t)ext;
      }
      w[0] = empty ? 0 : (int32_t)base;
    }
    rec[15] = (int32_t)(windowOf[g] << 2); // bits 0 and 1 are the flags set below
  }
  {
    // the b window of each distinct window, from the first record that has it
    // (records hold it at words 5..9): one pass over the slots
    std::vector<char> have(windowRep.size(), 0);
    for (size_t slot = 0; slot < slots.size(); ++slot) {
      if (slots[slot] < 0)
        continue;
      const size_t w = windowOf[(size_t)slots[slot]];
      if (have[w])
        continue;
      have[w] = 1;
      std::memcpy(host.data() + plan->offWindows + w * 8,
                  host.data() + plan->offGroups + slot * kGatherRecord + 5, 5 * sizeof(int32_t));
    }
  }
  for (int o = 0; o < 3; ++o) {
    gatherEntries(*ops[o], ops[o]->rowIndex, rows[o], rowDim[o],
                  host.data() + plan->offRows[o]);
    gatherEntries(*ops[o], ops[o]->colIndex, cols[o], colDim[o],
                  host.data() + plan->offCols[o]);
  }
  // Flags in word 15 of a set's first record.  Bit 0: the out windows of the
  // set's records follow each other element by element (and are not empty), so
  // the values one tile element has for neighbouring records are adjacent in
  // memory.  Bit 1: the same for the a windows, and every a element (all tile
  // rows, all of K) of every record is active, so the kernel may read them
  // without looking at the tables' indices.
  if (fuse >= 4) {
    // largest index each a entry needs along each dimension
    int32_t need[4] = {0, 0, 0, 0};
    bool nonneg = true;
    for (int axis = 0; axis < 2; ++axis) {
      const size_t n = axis ? cols[0] : rows[0];
      const int32_t *tab = host.data() + (axis ? plan->offCols[0] : plan->offRows[0]);
      for (size_t i = 0; i < n; ++i)
        for (int d = 0; d < 4; ++d) {
          const int32_t idx = tab[i * kGatherEntry + 1 + d];
          nonneg = nonneg && idx >= 0;
          need[d] = std::max(need[d], idx);
        }
    }
    for (size_t s0 = 0; s0 < slots.size(); s0 += fuse) {
      int32_t *rec0 = host.data() + plan->offGroups + s0 * kGatherRecord;
      bool runO = true, runA = nonneg;
      for (size_t i = 0; i < fuse; ++i) {
        const int32_t *ri = rec0 + i * kGatherRecord;
        if (slots[s0 + i] < 0) {
          runO = runA = false;
          break;
        }
        for (int d = 0; d < 4; ++d) {
          runO = runO && ri[11 + d] > 0;
          runA = runA && ri[1 + d] > need[d];
        }
        if (i > 0) {
          runO = runO && ri[10] == ri[10 - kGatherRecord] + 1;
          runA = runA && ri[0] == ri[0 - kGatherRecord] + 1;
        }
      }
      rec0[15] |= (runO ? 1 : 0) | (runA ? 2 : 0);
    }
  }
  if (dev->makeCurrent() ||
      HIP_CHECK(dev, hipMalloc((void **)&plan->tables, total * sizeof(int32_t)))) {
    delete plan;
    return nullptr;
  }
  const size_t packed = std::max<size_t>(
      (size_t)plan->nWindows * plan->kPad * plan->tnPad, 4);
  if (HIP_CHECK(dev, hipMemcpy(plan->tables, host.data(),
                               total * sizeof(int32_t), hipMemcpyHostToDevice)) ||
      HIP_CHECK(dev, hipMalloc((void **)&plan->bpack, packed * sizeof(float)))) {
    (void)hipFree(plan->tables);
    delete plan;
    return nullptr;
  }
  return plan;
}

int hcamdGatherGemmLaunchF32(OlQueue q, HcamdGatherGemm plan, const float *a,
                             const float *b, float *out) noexcept {
  return hcamdGatherGemmLaunch(q, plan, HCAMD_F32, a, b, out);
}

int hcamdGatherGemmLaunch(OlQueue q, HcamdGatherGemm plan, int elemType,
                          const void *a, const void *b, void *out) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  if (elemType != HCAMD_F32 && elemType != HCAMD_F16 && elemType != HCAMD_BF16) {
    dev->report("hcamdGatherGemmLaunch: unknown element type %d", elemType);
    return 1;
  }
  static const char *const kTypes[] = {"f32", "f16", "bf16"};
  const char *ty = kTypes[elemType];
  if (!plan || plan->device != dev) {
    dev->report("hcamdGatherGemmLaunch: the plan belongs to another device");
    return 1;
  }
  if (!a || !b || !out) {
    dev->report("hcamdGatherGemmLaunch: null pointer");
    return 1;
  }
  // Block edge of the kernel: the smallest of 8, 16, 32, 64 that holds the
  // tile of fuse * tm rows (64 for larger tiles, which are walked block by
  // block).  Blocks of 32 and 64 multiply on the matrix cores, the small ones
  // on the vector ALUs.  Variants: 1 m64, 2 m32, 3 t16, 4 t8, 5 t64, 6 t32
  // (t = vector ALUs); fusing four records needs m64, fusing two any but the
  // last two.
  const uint32_t side = std::max(plan->tm * plan->fuse, plan->tn);
  int variant = variantOf("gather");
  if (variant < 1 || variant > 6)
    variant = plan->fuse >= 4 ? 1
              : side <= 8     ? 4
              : side <= 16    ? 3
              : side <= 32    ? 2
                              : 1;
  if ((plan->fuse >= 4 && variant != 1) || (plan->fuse == 2 && variant > 4) ||
      (elemType != HCAMD_F32 && variant > 4)) {
    dev->report("hcamdGatherGemmLaunch: block shape %d is not built for %u "
                "fused records of type %s", variant, plan->fuse, ty);
    return 1;
  }
  static const char *const kShapes[] = {"m64", "m32", "t16", "t8", "t64", "t32"};
  char name[64];
  std::snprintf(name, sizeof(name), "hcamd_gather_gemm_%s_%s_g%u", ty,
                kShapes[variant - 1], plan->fuse);
  const size_t threads = (variant == 1 || variant == 5) ? 256 : 64;
  Kernel *kern = builtinKernel(dev, "gather", name);
  if (!kern)
    return 1;
  const int32_t *t = plan->tables;
  if (plan->k > 0) {
    // every distinct b tile once, then the products
    // 16-bit storage on the matrix-core blocks reads its b tiles in the
    // stored type, column by column
    const bool low = elemType != HCAMD_F32 && (variant == 1 || variant == 2);
    char packName[48];
    std::snprintf(packName, sizeof(packName), "hcamd_gather_pack_b_%s%s",
                  low ? "low_" : "", ty);
    Kernel *pack = builtinKernel(dev, "gather", packName);
    if (!pack)
      return 1;
    PackBArgs pb;
    pb.b = b;
    pb.bpack = plan->bpack;
    pb.windows = t + plan->offWindows;
    pb.b_rows = t + plan->offRows[1];
    pb.b_cols = t + plan->offCols[1];
    pb.k = plan->k;
    pb.tn = plan->tn;
    pb.k_pad = plan->kPad;
    pb.tn_pad = plan->tnPad;
    pb.n_windows = plan->nWindows;
    void *pparams[] = {&pb};
    const size_t per = (size_t)plan->kPad * plan->tnPad;
    const size_t pgrid[3] = {std::min<size_t>(ceilDiv(per, 256), 4096),
                             plan->nWindows, 1};
    const size_t pblock[3] = {256, 1, 1};
    if (launch(queue, pack, pgrid, pblock, pparams, 0))
      return 1;
  }
  GatherGemmArgs args;
  args.a = a;
  args.bpack = plan->bpack;
  args.out = out;
  args.groups = t + plan->offGroups;
  args.a_rows = t + plan->offRows[0];
  args.a_cols = t + plan->offCols[0];
  args.o_rows = t + plan->offRows[2];
  args.o_cols = t + plan->offCols[2];
  args.tm = plan->tm;
  args.tn = plan->tn;
  args.k = plan->k;
  args.n_groups = plan->nSets;
  args.per_xcd = (plan->nSets + 7) / 8;
  args.k_pad = plan->kPad;
  args.tn_pad = plan->tnPad;
  void *params[] = {&args};
  // y: the blocks of a tile (the kernel strides over them if there are more)
  const size_t edge = (variant == 1 || variant == 5)   ? 64
                      : (variant == 2 || variant == 6) ? 32
                      : variant == 3                   ? 16
                                                       : 8;
  const size_t tileBlocks = ceilDiv((size_t)plan->tm * plan->fuse, edge) *
                            ceilDiv((size_t)plan->tn, edge);
  const size_t grid[3] = {(size_t)args.per_xcd * 8,
                          std::min<size_t>(tileBlocks, 65535), 1};
  const size_t block[3] = {threads, 1, 1};
  return launch(queue, kern, grid, block, params, 0);
}

void hcamdGatherGemmRelease(HcamdGatherGemm plan) noexcept {
  if (!plan)
    return;
  if (!plan->device->makeCurrent()) {
    if (plan->tables)
      (void)hipFree(plan->tables);
    if (plan->bpack)
      (void)hipFree(plan->bpack);
  }
  delete plan;
}

// ---------------------------------------------------------------------------
// Elementwise expressions of gathered tiles
// ---------------------------------------------------------------------------
struct HcamdGatherMap_ {
  Device *device = nullptr;
  int32_t *tables = nullptr; // one device allocation: per operand starts[groups][4], index[elems][4]
  size_t offStarts[kMapMaxIn + 1] = {}, offIndex[kMapMaxIn + 1] = {};
  uint32_t shape[kMapMaxIn + 1][4] = {}, strides[kMapMaxIn + 1][4] = {};
  size_t nInputs = 0, nGroups = 0, tileElems = 0;
};

namespace {
// argument block of hcamd_gather_fmap (the same layout as in the device code)
struct GatherMapOperandDev {
  const int32_t *starts;
  const int32_t *index;
  uint32_t shape[4];
  uint32_t strides[4];
};
struct GatherMapArgs {
  const void *in[kMapMaxIn];
  void *out;
  GatherMapOperandDev op[kMapMaxIn + 1];
  uint32_t nIn, tileElems, chunks;
  uint32_t f16Mask, outType, storeAll, copyBytes, nInstr;
  HcamdMapInstr prog[48];
};
} // namespace

HcamdGatherMap hcamdGatherMapCreate(OlQueue q, const HcamdGatherMapOperand *operands, size_t nInputs,
                                    size_t nGroups, size_t tileElems) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return nullptr;
  Device *dev = queue->device;
  const char *who = "hcamdGatherMapCreate";
  if (!operands || nInputs < 1 || nInputs > kMapMaxIn || nGroups == 0 || tileElems == 0 ||
      nGroups > 0x7fffffffull || tileElems > ((size_t)1 << 24)) {
    dev->report("%s: %zu operands (1..%zu), %zu groups, %zu tile elements", who, nInputs, kMapMaxIn,
                nGroups, tileElems);
    return nullptr;
  }
  const size_t chunks = ceilDiv(tileElems, (size_t)256);
  if (nGroups * chunks > 0x7fffffffull) {
    dev->report("%s: %zu groups of %zu elements are more workgroups than a launch holds", who,
                nGroups, tileElems);
    return nullptr;
  }
  auto *plan = new (std::nothrow) HcamdGatherMap_;
  if (!plan) {
    dev->report("%s: out of host memory", who);
    return nullptr;
  }
  plan->device = dev;
  plan->nInputs = nInputs;
  plan->nGroups = nGroups;
  plan->tileElems = tileElems;
  size_t total = 0;
  for (size_t o = 0; o <= nInputs; ++o) {
    const HcamdGatherMapOperand &op = operands[o];
    if (op.ndim < 1 || op.ndim > 4 || !op.starts || !op.index) {
      dev->report("%s: operand %zu: rank %d or null table", who, o, op.ndim);
      delete plan;
      return nullptr;
    }
    size_t span = 1;
    for (int d = 0; d < 4; ++d) {
      const size_t n = d < op.ndim ? op.shape[d] : 1, st = d < op.ndim ? op.strides[d] : 0;
      if (n == 0 || n > 0x7fffffffull || st > 0x7fffffffull) {
        dev->report("%s: operand %zu: empty or larger than 2^31 along dimension %d", who, o, d);
        delete plan;
        return nullptr;
      }
      plan->shape[o][d] = (uint32_t)n;
      plan->strides[o][d] = (uint32_t)st;
      span += (n - 1) * st;
    }
    if (span > 0x7fffffffull) {
      dev->report("%s: operand %zu spans more than 2^31 elements", who, o);
      delete plan;
      return nullptr;
    }
    for (size_t g = 0; g < nGroups * (size_t)op.ndim; ++g)
      if (op.starts[g] < 0) {
        dev->report("%s: operand %zu: negative window start", who, o);
        delete plan;
        return nullptr;
      }
    plan->offStarts[o] = total;
    total += nGroups * 4;
    plan->offIndex[o] = total;
    total += tileElems * 4;
  }
  std::vector<int32_t> host;
  try {
    host.assign(total, 0);
  } catch (...) {
    dev->report("%s: out of host memory", who);
    delete plan;
    return nullptr;
  }
  for (size_t o = 0; o <= nInputs; ++o) {
    const HcamdGatherMapOperand &op = operands[o];
    for (size_t g = 0; g < nGroups; ++g)
      for (int d = 0; d < op.ndim; ++d)
        host[plan->offStarts[o] + g * 4 + d] = op.starts[g * op.ndim + d];
    for (size_t e = 0; e < tileElems; ++e)
      for (int d = 0; d < op.ndim; ++d)
        host[plan->offIndex[o] + e * 4 + d] = op.index[e * op.ndim + d];
  }
  if (dev->makeCurrent() ||
      HIP_CHECK(dev, hipMalloc(reinterpret_cast<void **>(&plan->tables), total * sizeof(int32_t)))) {
    delete plan;
    return nullptr;
  }
  if (HIP_CHECK(dev, hipMemcpy(plan->tables, host.data(), total * sizeof(int32_t), hipMemcpyHostToDevice))) {
    (void)hipFree(plan->tables);
    delete plan;
    return nullptr;
  }
  return plan;
}

int hcamdGatherMapLaunch(OlQueue q, HcamdGatherMap plan, const HcamdMapInstr *prog, size_t nInstr,
                         const void *const *inputs, const int *inputTypes, void *out, int outType,
                         int storeAll, size_t copyBytes) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  const char *who = "hcamdGatherMapLaunch";
  if (!plan || plan->device != dev || !inputs || !out) {
    dev->report("%s: null pointer, or a plan of another device", who);
    return 1;
  }
  GatherMapArgs a{};
  if (copyBytes) {
    if (copyBytes != 1 && copyBytes != 2 && copyBytes != 4 && copyBytes != 8) {
      dev->report("%s: copies move elements of 1, 2, 4 or 8 bytes", who);
      return 1;
    }
    a.copyBytes = (uint32_t)copyBytes;
  } else {
    if (!prog || !inputTypes || nInstr == 0 || nInstr > 48) {
      dev->report("%s: program of %zu instructions (1..48)", who, nInstr);
      return 1;
    }
    if (outType != HCAMD_F32 && outType != HCAMD_F16 && outType != HCAMD_U8) {
      dev->report("%s: unsupported output type %d", who, outType);
      return 1;
    }
    int sp = 0;
    for (size_t i = 0; i < nInstr; ++i) {
      const unsigned op = prog[i].op;
      if (op == HCAMD_FMAP_END || op >= HCAMD_FMAP_COUNT) {
        dev->report("%s: bad opcode %u at %zu", who, op, i);
        return 1;
      }
      if (op == HCAMD_FMAP_IN && prog[i].arg >= plan->nInputs) {
        dev->report("%s: operand %u at %zu (only %zu given)", who, prog[i].arg, i, plan->nInputs);
        return 1;
      }
      const bool push = op == HCAMD_FMAP_IN || op == HCAMD_FMAP_CONST;
      const bool select = op == HCAMD_FMAP_SELECT; // three entries in, one out
      const bool unary = op >= HCAMD_FMAP_NEG && !select && op != HCAMD_FMAP_MERGE; // (MERGE: two in, one out)
      if (sp < (push ? 0 : unary ? 1 : select ? 3 : 2)) {
        dev->report("%s: stack underflow at %zu", who, i);
        return 1;
      }
      sp += push ? 1 : unary ? 0 : select ? -2 : -1;
      if (sp > 4) {
        dev->report("%s: stack deeper than 4 at %zu", who, i);
        return 1;
      }
      a.prog[i] = prog[i];
    }
    if (sp != 1) {
      dev->report("%s: program leaves %d values, expected 1", who, sp);
      return 1;
    }
    a.nInstr = (uint32_t)nInstr;
    a.outType = outType == HCAMD_F32 ? 0u : outType == HCAMD_F16 ? 1u : 2u;
    if (storeAll < 0 || storeAll > 2) {
      dev->report("%s: storeAll is 0, 1 or 2", who);
      return 1;
    }
    a.storeAll = (uint32_t)storeAll;
  }
  for (size_t i = 0; i <= plan->nInputs; ++i) {
    if (i < plan->nInputs) {
      if (!inputs[i]) {
        dev->report("%s: null pointer", who);
        return 1;
      }
      if (!copyBytes && inputTypes[i] != HCAMD_F32 && inputTypes[i] != HCAMD_F16 &&
          inputTypes[i] != HCAMD_I32) {
        dev->report("%s: unsupported operand type %d", who, inputTypes[i]);
        return 1;
      }
      a.in[i] = inputs[i];
      if (!copyBytes && inputTypes[i] == HCAMD_F16)
        a.f16Mask |= 1u << i;
      if (!copyBytes && inputTypes[i] == HCAMD_I32)
        a.f16Mask |= 1u << (8 + i); // converted to fp32 when read
    }
    a.op[i].starts = plan->tables + plan->offStarts[i];
    a.op[i].index = plan->tables + plan->offIndex[i];
    for (int d = 0; d < 4; ++d) {
      a.op[i].shape[d] = plan->shape[i][d];
      a.op[i].strides[d] = plan->strides[i][d];
    }
  }
  a.out = out;
  a.nIn = (uint32_t)plan->nInputs;
  a.tileElems = (uint32_t)plan->tileElems;
  a.chunks = (uint32_t)ceilDiv(plan->tileElems, (size_t)256);
  void *args[] = {&a};
  return launch1d(queue, "fmap", "hcamd_gather_fmap", plan->nGroups * a.chunks, 256, args);
}

void hcamdGatherMapRelease(HcamdGatherMap plan) noexcept {
  if (!plan)
    return;
  if (!plan->device->makeCurrent() && plan->tables)
    (void)hipFree(plan->tables);
  delete plan;
}

int hcamdLaunchSoftmaxF32(OlQueue q, const float *x, size_t ldx, float *y,
                          size_t ldy, size_t rows, size_t cols) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  if (rows == 0 || cols == 0)
    return 0;
  if (!x || !y) {
    dev->report("hcamdLaunchSoftmaxF32: null pointer");
    return 1;
  }
  if (rows > 1 && (ldx < cols || ldy < cols)) {
    dev->report("hcamdLaunchSoftmaxF32: leading dimension smaller than cols");
    return 1;
  }
  if (rows > 0x7fffffffull) {
    dev->report("hcamdLaunchSoftmaxF32: too many rows");
    return 1;
  }
  void *args[] = {&x, &ldx, &y, &ldy, &rows, &cols};
  const int variant = variantOf("softmax");
  const bool vec_ok = aligned16(x) && aligned16(y) &&
                      (rows == 1 || (ldx % 4 == 0 && ldy % 4 == 0));
  if (variant == 1)
    return launch1d(queue, "softmax", "hcamd_softmax_f32_stream", rows, 256,
                    args);
  if (cols > 32768 || (cols > 16384 && variant == 2))
    // longer than the registers of a workgroup: two sweeps, online maximum / sum
    // (parking the tail of such a row in LDS, one 1024-lane workgroup per CU,
    // measured no faster)
    return launch1d(queue, "softmax", "hcamd_softmax_f32_online", rows, 1024,
                    args);
  if (cols > 16384)
    // 1024 lanes per row, 32 elements per lane in registers
    return launch1d(queue, "softmax", "hcamd_softmax_f32_s1024_e32", rows, 1024,
                    args);
  if (!vec_ok) {
    // rows that do not start on 16-byte boundaries: register-resident with
    // 4-byte accesses
    const char *scalar = cols <= 1024   ? "hcamd_softmax_f32_s256_e4"
                         : cols <= 2048 ? "hcamd_softmax_f32_s256_e8"
                         : cols <= 4096 ? "hcamd_softmax_f32_s256_e16"
                         : cols <= 8192 ? "hcamd_softmax_f32_s256_e32"
                                        : "hcamd_softmax_f32_s256_e64";
    return launch1d(queue, "softmax", scalar, rows, 256, args);
  }
  const char *name;
  size_t groups = rows;
  if (cols <= 1024) {
    name = cols <= 256   ? "hcamd_softmax_f32_w64_v1"
           : cols <= 512 ? "hcamd_softmax_f32_w64_v2"
                         : "hcamd_softmax_f32_w64_v4";
    groups = ceilDiv(rows, 4);
  } else if (cols <= 2048) {
    name = (cols == 2048 && variant != 2) ? "hcamd_softmax_f32_g256_v2_full"
                                          : "hcamd_softmax_f32_g256_v2";
  } else if (cols <= 4096) {
    name = (cols == 4096 && variant != 2) ? "hcamd_softmax_f32_g256_v4_full"
                                          : "hcamd_softmax_f32_g256_v4";
  } else if (cols <= 8192) {
    const size_t cus = (size_t)computeUnitsOf(dev);
    if (cols == 8192 && variant == 0)
      // full rows: 1024 lanes per row, two 16-byte words per lane
      return launch1d(queue, "softmax", "hcamd_softmax_f32_g1024_v2_full_nt", rows, 1024,
                      args);
    if (cols == 8192 && variant == 11)
      // the same with one exchange of (maximum, sum) pairs between the waves
      return launch1d(queue, "softmax", "hcamd_softmax_f32_g1024_v2_one_exchange_nt", rows, 1024,
                      args);
    if (cols == 8192 && ((variant == 10 && rows >= 8 * cus) ||
                         (variant >= 5 && variant <= 9))) {
      // Full rows and enough of them: the persistent kernel, a fixed number of
      // workgroups per compute unit, each prefetching its next row.
      static const int per_cu[] = {4, 8, 2, 6, 3};
      name = "hcamd_softmax_f32_p256_v8_nt";
      groups = std::min<size_t>(rows, cus * per_cu[variant >= 5 ? variant - 5 : 0]);
    } else if (variant == 4) {
      name = cols == 8192 ? "hcamd_softmax_f32_g256_v8_full_nt_acc"
                          : "hcamd_softmax_f32_g256_v8_acc";
    } else {
      name = (cols == 8192 && variant != 2)
                 ? (variant == 3 ? "hcamd_softmax_f32_g256_v8_full"
                                 : "hcamd_softmax_f32_g256_v8_full_nt")
                 : "hcamd_softmax_f32_g256_v8";
    }
  } else {
    name = "hcamd_softmax_f32_g256_v16";
  }
  return launch1d(queue, "softmax", name, groups, 256, args);
}

int hcamdLaunchQuantizeF16I8(OlQueue q, const void *x, size_t ldx, int8_t *qout,
                             size_t ldq, float *scale, size_t rows,
                             size_t cols) noexcept {
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  if (rows == 0)
    return 0;
  if (!x || !qout || !scale) {
    dev->report("hcamdLaunchQuantizeF16I8: null pointer");
    return 1;
  }
  if (cols == 0) {
    // no elements: the absmax of an empty row is taken as 0
    return hcamdFill32(q, scale, 0u, rows);
  }
  if (rows > 1 && (ldx < cols || ldq < cols)) {
    dev->report("hcamdLaunchQuantizeF16I8: leading dimension smaller than cols");
    return 1;
  }
  if (rows > 0x7fffffffull) {
    dev->report("hcamdLaunchQuantizeF16I8: too many rows");
    return 1;
  }
  void *args[] = {&x, &ldx, &qout, &ldq, &scale, &rows, &cols};
  const int variant = variantOf("quantize");
  const bool vec_ok = aligned16(x) && aligned16(qout) &&
                      (rows == 1 || (ldx % 8 == 0 && ldq % 16 == 0));
  if (variant == 0 && cols > 2048 && cols <= 4096 && cols % 8 == 0 && aligned16(x) &&
      reinterpret_cast<uintptr_t>(qout) % 8 == 0 && (rows == 1 || (ldx % 8 == 0 && ldq % 8 == 0))) {
    // 16-byte words dealt to the lanes one by one (the accesses of a plain copy:
    // 16-byte loads, 8-byte stores), two rows per workgroup of 512 lanes
    const bool full = cols == 4096 && rows % 2 == 0;
    return launch1d(queue, "quantize",
                    full ? "hcamd_quant_f16_i8_c256x2_w2_full_nt"
                         : "hcamd_quant_f16_i8_c256x2_w2_nt",
                    ceilDiv(rows, (size_t)2), 512, args);
  }
  if (!vec_ok && variant != 1 && cols <= 32768) {
    // rows that cannot be walked in 16-byte pieces: register-resident with the
    // widest access the leading dimensions and base addresses allow
    const uintptr_t ax = reinterpret_cast<uintptr_t>(x), aq = reinterpret_cast<uintptr_t>(qout);
    const bool one_row = rows == 1;
    const char *small = nullptr;
    if (ax % 8 == 0 && aq % 4 == 0 && (one_row || (ldx % 4 == 0 && ldq % 4 == 0)))
      small = cols <= 4096    ? "hcamd_quant_f16_i8_s4_e4"
              : cols <= 8192  ? "hcamd_quant_f16_i8_s4_e8"
              : cols <= 16384 ? "hcamd_quant_f16_i8_s4_e16"
                              : "hcamd_quant_f16_i8_s4_e32";
    else if (ax % 4 == 0 && aq % 2 == 0 && (one_row || (ldx % 2 == 0 && ldq % 2 == 0)))
      small = cols <= 4096    ? "hcamd_quant_f16_i8_s2_e8"
              : cols <= 8192  ? "hcamd_quant_f16_i8_s2_e16"
              : cols <= 16384 ? "hcamd_quant_f16_i8_s2_e32"
                              : "hcamd_quant_f16_i8_s2_e64";
    else if (cols <= 16384)
      small = cols <= 4096   ? "hcamd_quant_f16_i8_s1_e16"
              : cols <= 8192 ? "hcamd_quant_f16_i8_s1_e32"
                             : "hcamd_quant_f16_i8_s1_e64";
    if (small)
      return launch1d(queue, "quantize", small, rows, 256, args);
  }
  if (!vec_ok || cols > 32768 || variant == 1)
    return launch1d(queue, "quantize", "hcamd_quant_f16_i8_stream", rows, 256,
                    args);
  const char *name;
  size_t groups = rows;
  bool per_wave = false;
  size_t rows_per_group = 1;
  if (cols <= 1024) {
    name = "hcamd_quant_f16_i8_w64_v1";
    per_wave = true;
  } else if (cols <= 2048) {
    name = "hcamd_quant_f16_i8_w64_v2";
    per_wave = true;
  } else if (cols <= 4096) {
    switch (variant) {
    case 2: name = "hcamd_quant_f16_i8_w64_v4"; per_wave = true; break;
    case 3: name = "hcamd_quant_f16_i8_g256_v1"; break;
    case 4: name = "hcamd_quant_f16_i8_w64_v4_nt"; per_wave = true; break;
    case 5: name = "hcamd_quant_f16_i8_g256_v1_div"; break;
    case 6: name = "hcamd_quant_f16_i8_w64_v4_div"; per_wave = true; break;
    case 7: name = "hcamd_quant_f16_i8_g128_v2_nt"; rows_per_group = 2; break;
    default: name = "hcamd_quant_f16_i8_g256_v1_nt"; break;
    }
  } else if (cols <= 8192) {
    name = "hcamd_quant_f16_i8_g256_v2";
  } else if (cols <= 16384) {
    name = "hcamd_quant_f16_i8_g256_v4";
  } else {
    name = "hcamd_quant_f16_i8_g256_v8";
  }
  if (per_wave)
    rows_per_group = 4;
  groups = ceilDiv(rows, rows_per_group);
  // variants 8..11: persistent kernel for rows of exactly 4096 columns, with
  // 4 / 8 / 6 / 12 workgroups per CU
  if (cols == 4096 && variant >= 8 && variant <= 11) {
    static const size_t per_cu[] = {4, 8, 6, 12};
    name = "hcamd_quant_f16_i8_p256_v1_nt";
    groups = std::min(rows, (size_t)computeUnitsOf(dev) * per_cu[variant - 8]);
  }
  return launch1d(queue, "quantize", name, groups, 256, args);
}

namespace {
// Shared by the bf16 and fp16 entry points; `half` selects the fp16 kernels.
int launchGemm(OlQueue q, bool half, const void *a, size_t lda, const void *bt,
               size_t ldb, void *c, size_t ldc, size_t m, size_t n, size_t k) {
  const char *who = half ? "hcamdLaunchGemmF16" : "hcamdLaunchGemmBF16";
  auto *queue = static_cast<Queue *>(q);
  if (!queue)
    return 1;
  Device *dev = queue->device;
  if (m == 0 || n == 0)
    return 0;
  if (!a || !bt || !c) {
    dev->report("%s: null pointer", who);
    return 1;
  }
  if (k == 0) {
    dev->report("%s: K must be at least 1", who);
    return 1;
  }
  if ((m > 1 && lda < k) || (n > 1 && ldb < k) || (m > 1 && ldc < n)) {
    dev->report("%s: leading dimension too small", who);
    return 1;
  }
  if (m > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull) {
    dev->report("%s: dimension exceeds 2^31-1", who);
    return 1;
  }
  int M = (int)m, N = (int)n, K = (int)k;
  void *args[] = {&a, &lda, &bt, &ldb, &c, &ldc, &M, &N, &K};

  struct Tiled {
    const char *name;
    int bm, bn, threads;
  };
#ifdef HCAMD_PROBES
#define HCAMD_PROBE_NAME(n) n
#else
#define HCAMD_PROBE_NAME(n) nullptr // not in this build (and hcamdSetVariant refuses the number)
#endif
  static const Tiled tiled[] = {
      {"hcamd_gemm_bf16_256x256_w2x4_s0", 256, 256, 512}, // 1
      {"hcamd_gemm_bf16_256x256_w2x4_s1", 256, 256, 512},
      {"hcamd_gemm_bf16_256x256_w4x2_s0", 256, 256, 512},
      {"hcamd_gemm_bf16_128x128_w2x2_s0", 128, 128, 256},
      {"hcamd_gemm_bf16_256x128_w2x2_s0", 256, 128, 256},
      {nullptr, 0, 0, 0}, // 6: the general kernel
      {"hcamd_gemm_bf16_p256x256_w2x4", 256, 256, 512}, // 7
      {"hcamd_gemm_bf16_p256x256_w4x2", 256, 256, 512},
      {"hcamd_gemm_bf16_p128x128_w2x2", 128, 128, 256},
      {"hcamd_gemm_bf16_p256x128_w2x2", 256, 128, 256},
      {"hcamd_gemm_bf16_p32_256x256_w2x4", 256, 256, 512}, // 11
      {"hcamd_gemm_bf16_p32_256x256_w4x2", 256, 256, 512},
      {nullptr, 0, 0, 0}, // 13: the edge-capable kernel (chosen below)
      {"hcamd_gemm_bf16_p256x256_w2x4_direct", 256, 256, 512}, // 14: 8-byte stores from the accumulators
      {"hcamd_gemm_bf16_p256x256_w2x4_lds", 256, 256, 512},    // 15: through LDS, plain stores
      {"hcamd_gemm_bf16_p256x256_w2x4_prio", 256, 256, 512},   // 16: raised priority in the MFMA bursts
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_mfma_only"), 256, 256, 512},      // 17: measurement only, output is not the product
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_no_vmwait"), 256, 256, 512},      // 18..21: likewise
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_no_barrier"), 256, 256, 512},
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_no_ldsread"), 256, 256, 512},
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_no_loads"), 256, 256, 512},
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_loads_to_regs"), 256, 256, 512}, // 22
      {"hcamd_gemm_bf16_p256x256_w2x4_stage_a", 256, 256, 512},     // 23: A panel through registers
      {"hcamd_gemm_bf16_p256x256_w2x4_hinted", 256, 256, 512},      // 24: half-step order left to the compiler
      {"hcamd_gemm_bf16_p256x256_w2x4_loads_early", 256, 256, 512}, // 25: loads in the first half of the MFMAs
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_b_direct"), 256, 256, 512},            // 26: measurement only
      {"hcamd_gemm_bf16_p256x256_w2x2", 256, 256, 256},             // 27: four waves, 128 x 128 each
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_no_stores"), 256, 256, 512}, // 28: measurement only
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_two_tiles"), 256, 256, 512}, // 29: measurement only
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_w2x2_reads48"), 256, 256, 256}, // 30..32: other hand orders of 27
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_w2x2_loads2"), 256, 256, 256},  //         (the product, measurement builds only)
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_w2x2_a_inner"), 256, 256, 256},
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_mfma16_direct"), 256, 256, 512}, // 33, 34: measurement only
      {HCAMD_PROBE_NAME("hcamd_gemm_bf16_probe_mfma32_direct"), 256, 256, 512},
  };
  constexpr int kGeneral = 6;
  constexpr int kFirstPipelined = 7; // variants from here need K >= 128
  constexpr int kNumTiled = sizeof(tiled) / sizeof(tiled[0]);
  const int variant = variantOf("gemm");
  const bool vec_ok = aligned16(a) && aligned16(bt) && aligned16(c) &&
                      lda % 8 == 0 && ldb % 8 == 0 && ldc % 4 == 0 &&
                      k % 64 == 0;
  const Tiled *pick = nullptr;
  static const Tiled half256 = {"hcamd_gemm_f16_p256x256_w2x4", 256, 256, 512};
  static const Tiled half128 = {"hcamd_gemm_f16_p128x128_w2x2", 128, 128, 256};
  if (half) {
    if (vec_ok && k >= 128 && variant != kGeneral) {
      if (m % 256 == 0 && n % 256 == 0)
        pick = &half256;
      else if (m % 128 == 0 && n % 128 == 0)
        pick = &half128;
    }
  } else if (vec_ok && variant != kGeneral) {
    if (variant >= 1 && variant <= kNumTiled) {
      const Tiled &t = tiled[variant - 1];
      if (t.name && m % t.bm == 0 && n % t.bn == 0 &&
          (variant < kFirstPipelined || k >= 128))
        pick = &t;
    } else {
      // default: the pipelined 256 x 256 kernel; smaller or K < 128 shapes fall
      // back to the simpler tiled kernels
      if (m % 256 == 0 && n % 256 == 0 && k >= 128)
        pick = &tiled[kFirstPipelined - 1];
      else if (m % 256 == 0 && n % 256 == 0)
        pick = &tiled[0];
      else if (m % 128 == 0 && n % 128 == 0 && k >= 128)
        pick = &tiled[8];
      else if (m % 128 == 0 && n % 128 == 0)
        pick = &tiled[3];
    }
  }
  // The whole-tile pipelined kernels address their panels with 32-bit byte
  // offsets from the tile's first row (buffer loads): rows further apart than
  // that go to the edge-capable build, which uses 64-bit pointers.
  if (pick && pick - tiled >= kFirstPipelined - 1 &&
      ((size_t)(pick->bm - 1) * lda + k) * 2 >= ((size_t)1 << 31))
    pick = nullptr;
  if (pick && (pick == &half256 || pick == &half128 || pick - tiled >= kFirstPipelined - 1) &&
      ((size_t)(pick->bn - 1) * ldb + k) * 2 >= ((size_t)1 << 31))
    pick = nullptr;
  if (pick && (pick == &half256 || pick == &half128) &&
      ((size_t)(pick->bm - 1) * lda + k) * 2 >= ((size_t)1 << 31))
    pick = nullptr;
  // Shapes the whole-tile kernels cannot take (M or N not a multiple of the
  // tile, K not a multiple of 64) go to the edge-capable build of the pipelined
  // kernel as long as the panels can be fetched in 16-byte pieces; only what
  // is left (odd K or leading dimensions, K <= 64, misaligned A / Bt) takes the
  // general kernel.  Variant 13 forces the edge kernel, 6 the general one.
  static const Tiled edge[2][2] = {
      {{"hcamd_gemm_bf16_p256x256_w2x4_edge", 256, 256, 512},
       {"hcamd_gemm_bf16_p128x128_w2x2_edge", 128, 128, 256}},
      {{"hcamd_gemm_f16_p256x256_w2x4_edge", 256, 256, 512},
       {"hcamd_gemm_f16_p128x128_w2x2_edge", 128, 128, 256}}};
  const bool edge_ok = aligned16(a) && aligned16(bt) && lda % 8 == 0 &&
                       ldb % 8 == 0 && k % 8 == 0 && k > 64 &&
                       (reinterpret_cast<uintptr_t>(c) & 1) == 0;
  bool ragged = false;
  if (edge_ok && variant != kGeneral && (!pick || variant == 13)) {
    // the smaller tile when the larger one would leave most CUs idle
    const size_t big = ceilDiv(m, (size_t)256) * ceilDiv(n, (size_t)256);
    pick = &edge[half ? 1 : 0][big >= (size_t)computeUnitsOf(dev) / 2 ? 0 : 1];
    ragged = true;
  }
  if (pick) {
    Kernel *kn = builtinKernel(dev, "gemm", pick->name);
    if (!kn)
      return 1;
    const size_t grid[3] = {ragged ? ceilDiv(m, (size_t)pick->bm) * ceilDiv(n, (size_t)pick->bn)
                                   : (m / pick->bm) * (n / pick->bn),
                            1, 1};
    const size_t block[3] = {(size_t)pick->threads, 1, 1};
    return launch(queue, kn, grid, block, args, 0);
  }
  Kernel *kn = builtinKernel(dev, "gemm", half ? "hcamd_gemm_f16_general"
                                               : "hcamd_gemm_bf16_general");
  if (!kn)
    return 1;
  const size_t gy = ceilDiv(m, 64);
  if (gy > 65535) {
    dev->report("%s: M too large for the general kernel", who);
    return 1;
  }
  const size_t grid[3] = {ceilDiv(n, 64), gy, 1};
  const size_t block[3] = {256, 1, 1};
  return launch(queue, kn, grid, block, args, 0);
}
} // namespace

int hcamdLaunchGemmBF16(OlQueue q, const void *a, size_t lda, const void *bt,
                        size_t ldb, void *c, size_t ldc, size_t m, size_t n,
                        size_t k) noexcept {
  return launchGemm(q, false, a, lda, bt, ldb, c, ldc, m, n, k);
}

int hcamdLaunchGemmF16(OlQueue q, const void *a, size_t lda, const void *bt,
                       size_t ldb, void *c, size_t ldc, size_t m, size_t n,
                       size_t k) noexcept {
  return launchGemm(q, true, a, lda, bt, ldb, c, ldc, m, n, k);
}

} // extern "C"

// Runtime half of libcaten_hip.so: device/stream, caching allocator, copies,
// hipRTC compilation, module loading and kernel launch.  This is what a Caten
// HipBuffer / HipRuntime / Hip-Renderer calls through CFFI; it mirrors the slots
// Caten's Metal backend fills with objc_msgSend (source/byoc/metal.lisp:103-154,
// 252-345) and its CLANG backend with gcc + dlopen (source/byoc/clang.lisp:127-226).
#include <hip/hiprtc.h>
#include <stdarg.h>
#include <string.h>

#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace cthip {

static thread_local char g_err[2048] = "";
static char g_err_shared[2048] = "";

State &state() {
  static State s;
  return s;
}

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  memcpy(g_err_shared, g_err, sizeof(g_err));
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  memcpy(g_err_shared, g_err, sizeof(g_err));
  return code;
}

// ------------------------------------------------------------------
// Caching allocator.  Every Caten buffer whose shape mentions the symbolic
// `s`/`n` is closed and re-opened on each decode step
// (source/runtime/runtime.lisp:248-259), so open/close must not reach the driver.
// Blocks are binned by size class (256 B granules up to 4 KiB, then 8 classes per
// power of two); a freed block is reused only for the same class.
// ------------------------------------------------------------------
struct Allocator {
  std::mutex mu;
  std::unordered_map<void *, size_t> live;            // ptr -> class bytes
  std::map<size_t, std::vector<void *>> cache;        // class bytes -> free blocks
  size_t live_bytes = 0, cached_bytes = 0, driver_allocs = 0;
};
static Allocator &allocator() {
  static Allocator a;
  return a;
}

static size_t size_class(size_t bytes) {
  if (bytes <= 256) return 256;
  if (bytes <= 4096) return (bytes + 255) & ~(size_t)255;
  size_t p = 4096;
  while (p * 2 < bytes) p *= 2;  // p < bytes <= 2p
  size_t step = p / 8;
  return p + (bytes - p + step - 1) / step * step;
}

__global__ void k_fill_zero(uint4 *p, size_t n16) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  uint4 z = {0u, 0u, 0u, 0u};
  for (; i < n16; i += stride) p[i] = z;
}

static int zero_fill(void *p, size_t bytes) {  // bytes is a multiple of 256
  size_t n16 = bytes / 16;
  size_t blocks = (n16 + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(k_fill_zero, dim3((unsigned)blocks), dim3(256), 0, state().stream, (uint4 *)p, n16);
  CTHIP_LAUNCH_CHECK();
  return 0;
}

// pinned staging ring for small host->device copies
struct Staging {
  static const int kSlots = 8;
  static const size_t kSlotBytes = 64 * 1024;
  char *base = nullptr;
  hipEvent_t ev[kSlots] = {};
  bool used[kSlots] = {};
  int next = 0;
};
static Staging &staging() {
  static Staging s;
  return s;
}

}  // namespace cthip

using namespace cthip;

extern "C" {

const char *cthip_last_error(void) { return g_err_shared; }

int cthip_init(int device) {
  State &s = state();
  if (s.inited) {
    if (s.device == device) return 0;
    return fail(CTHIP_E_STATE, "cthip_init: already initialised on device %d", s.device);
  }
  int n = 0;
  CTHIP_CHECK(hipGetDeviceCount(&n));
  if (device < 0 || device >= n) return fail(CTHIP_E_BAD_ARG, "cthip_init: device %d of %d", device, n);
  CTHIP_CHECK(hipSetDevice(device));
  hipDeviceProp_t prop;
  CTHIP_CHECK(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(CTHIP_E_UNSUPPORTED, "cthip_init: device is %s; this library is built for gfx950 only", prop.gcnArchName);
  s.compute_units = prop.multiProcessorCount;
  CTHIP_CHECK(hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking));
  CTHIP_CHECK(hipEventCreate(&s.ev0));
  CTHIP_CHECK(hipEventCreate(&s.ev1));
  Staging &st = staging();
  CTHIP_CHECK(hipHostMalloc((void **)&st.base, Staging::kSlots * Staging::kSlotBytes, hipHostMallocDefault));
  for (int i = 0; i < Staging::kSlots; i++) {
    CTHIP_CHECK(hipEventCreateWithFlags(&st.ev[i], hipEventDisableTiming));
    st.used[i] = false;
  }
  {
    int rc = matmul_scratch_init(device);
    if (rc) return rc;
  }
  s.device = device;
  s.inited = true;
  return 0;
}

int cthip_shutdown(void) {
  State &s = state();
  if (!s.inited) return 0;
  CTHIP_CHECK(hipStreamSynchronize(s.stream));
  cthip_cache_trim();
  Allocator &a = allocator();
  {
    std::lock_guard<std::mutex> lk(a.mu);
    for (auto &kv : a.live) (void)hipFree(kv.first);
    a.live.clear();
    a.live_bytes = 0;
  }
  Staging &st = staging();
  for (int i = 0; i < Staging::kSlots; i++) (void)hipEventDestroy(st.ev[i]);
  (void)hipHostFree(st.base);
  st.base = nullptr;
  (void)hipEventDestroy(s.ev0);
  (void)hipEventDestroy(s.ev1);
  (void)hipStreamDestroy(s.stream);
  s = State();
  return 0;
}

int cthip_device_info(char *name, int name_cap, int *compute_units, int *wave_size, size_t *lds_bytes,
                      size_t *mem_bytes) {
  CTHIP_REQUIRE_INIT();
  hipDeviceProp_t prop;
  CTHIP_CHECK(hipGetDeviceProperties(&prop, state().device));
  if (name && name_cap > 0) snprintf(name, name_cap, "%s (%s)", prop.name, prop.gcnArchName);
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (wave_size) *wave_size = prop.warpSize;
  if (lds_bytes) *lds_bytes = prop.sharedMemPerBlock;
  if (mem_bytes) *mem_bytes = prop.totalGlobalMem;
  return 0;
}

}  // extern "C"

// true when a kernel may dereference p: device, managed or pinned host memory.  Pageable host memory handed
// to a kernel would fault the GPU, so entry points that take device pointers from callers check first.
bool cthip::device_readable(const void *p) {
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
    (void)hipGetLastError();  // the failed query must not be reported by the next launch check
    return false;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged || attr.type == hipMemoryTypeHost;
}

// a block of the caching allocator with whatever its last owner left in it (temporaries that are
// fully written before they are read); released with cthip_free like any other block
int cthip::alloc_scratch(void **out, size_t bytes) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(out != nullptr);
  size_t cls = size_class(bytes);
  Allocator &a = allocator();
  void *p = nullptr;
  {
    std::lock_guard<std::mutex> lk(a.mu);
    auto it = a.cache.find(cls);
    if (it != a.cache.end() && !it->second.empty()) {
      p = it->second.back();
      it->second.pop_back();
      a.cached_bytes -= cls;
    }
  }
  if (!p) {
    hipError_t e = hipMalloc(&p, cls);
    if (e != hipSuccess) {  // give cached blocks back to the driver and retry once
      (void)hipGetLastError();
      cthip_cache_trim();
      e = hipMalloc(&p, cls);
    }
    if (e != hipSuccess) return fail((int)e, "cthip_alloc: hipMalloc(%zu) -> %s", cls, hipGetErrorString(e));
    std::lock_guard<std::mutex> lk(a.mu);
    a.driver_allocs++;
  }
  {
    std::lock_guard<std::mutex> lk(a.mu);
    a.live[p] = cls;
    a.live_bytes += cls;
  }
  *out = p;
  return 0;
}

extern "C" {

int cthip_alloc(void **out, size_t bytes) {
  int rc = cthip::alloc_scratch(out, bytes);
  if (rc) return rc;
  return zero_fill(*out, size_class(bytes));
}

int cthip_free(void *p) {
  if (!p) return 0;
  CTHIP_REQUIRE_INIT();
  Allocator &a = allocator();
  std::lock_guard<std::mutex> lk(a.mu);
  auto it = a.live.find(p);
  if (it == a.live.end()) return fail(CTHIP_E_BAD_ARG, "cthip_free: %p is not a live block of this allocator", p);
  size_t cls = it->second;
  a.live.erase(it);
  a.live_bytes -= cls;
  // Work queued earlier on the in-order stream may still read the block; any later
  // owner's work is queued after it on the same stream, so reuse is safe.
  a.cache[cls].push_back(p);
  a.cached_bytes += cls;
  return 0;
}

int cthip_cache_trim(void) {
  CTHIP_REQUIRE_INIT();
  CTHIP_CHECK(hipStreamSynchronize(state().stream));
  Allocator &a = allocator();
  std::lock_guard<std::mutex> lk(a.mu);
  for (auto &kv : a.cache)
    for (void *p : kv.second) (void)hipFree(p);
  a.cache.clear();
  a.cached_bytes = 0;
  return 0;
}

int cthip_cache_stats(size_t *live_bytes, size_t *cached_bytes, size_t *driver_allocs) {
  Allocator &a = allocator();
  std::lock_guard<std::mutex> lk(a.mu);
  if (live_bytes) *live_bytes = a.live_bytes;
  if (cached_bytes) *cached_bytes = a.cached_bytes;
  if (driver_allocs) *driver_allocs = a.driver_allocs;
  return 0;
}

int cthip_h2d(void *dst, const void *src, size_t bytes) {
  CTHIP_REQUIRE_INIT();
  if (bytes == 0) return 0;
  CTHIP_ARG(dst != nullptr && src != nullptr);
  State &s = state();
  Staging &st = staging();
  if (bytes <= Staging::kSlotBytes) {
    int i = st.next;
    st.next = (st.next + 1) % Staging::kSlots;
    if (st.used[i]) CTHIP_CHECK(hipEventSynchronize(st.ev[i]));
    char *slot = st.base + (size_t)i * Staging::kSlotBytes;
    memcpy(slot, src, bytes);
    CTHIP_CHECK(hipMemcpyAsync(dst, slot, bytes, hipMemcpyHostToDevice, s.stream));
    CTHIP_CHECK(hipEventRecord(st.ev[i], s.stream));
    st.used[i] = true;
    return 0;
  }
  // large transfers (weights): the driver stages pageable memory itself; the call
  // returns once the source has been consumed
  CTHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s.stream));
  CTHIP_CHECK(hipStreamSynchronize(s.stream));
  return 0;
}

int cthip_d2h(void *dst, const void *src, size_t bytes) {
  CTHIP_REQUIRE_INIT();
  State &s = state();
  if (bytes) {
    CTHIP_ARG(dst != nullptr && src != nullptr);
    CTHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s.stream));
  }
  CTHIP_CHECK(hipStreamSynchronize(s.stream));
  return 0;
}

int cthip_d2d(void *dst, const void *src, size_t bytes) {
  CTHIP_REQUIRE_INIT();
  if (bytes == 0) return 0;
  CTHIP_ARG(dst != nullptr && src != nullptr);
  CTHIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, state().stream));
  return 0;
}

int cthip_memset(void *dst, int byte, size_t bytes) {
  CTHIP_REQUIRE_INIT();
  if (bytes == 0) return 0;
  CTHIP_ARG(dst != nullptr);
  CTHIP_CHECK(hipMemsetAsync(dst, byte, bytes, state().stream));
  return 0;
}

int cthip_sync(void) {
  CTHIP_REQUIRE_INIT();
  CTHIP_CHECK(hipStreamSynchronize(state().stream));
  return 0;
}

void *cthip_stream(void) { return (void *)state().stream; }

int cthip_timer_start(void) {
  CTHIP_REQUIRE_INIT();
  CTHIP_CHECK(hipEventRecord(state().ev0, state().stream));
  return 0;
}

int cthip_timer_stop(float *ms) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(ms != nullptr);
  CTHIP_CHECK(hipEventRecord(state().ev1, state().stream));
  CTHIP_CHECK(hipEventSynchronize(state().ev1));
  CTHIP_CHECK(hipEventElapsedTime(ms, state().ev0, state().ev1));
  return 0;
}

// ------------------------------------------------------------------ hipRTC
int cthip_compile(const char *hip_source, const char *arch, void **code, size_t *code_size, char **log) {
  if (log) *log = nullptr;
  if (!hip_source || !code || !code_size) return fail(CTHIP_E_BAD_ARG, "cthip_compile: null argument");
  *code = nullptr;
  *code_size = 0;
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, hip_source, "caten_kernels.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return fail((int)r, "cthip_compile: hiprtcCreateProgram -> %s", hiprtcGetErrorString(r));
  std::string archopt = std::string("--offload-arch=") + (arch && *arch ? arch : "gfx950");
  const char *opts[] = {archopt.c_str(), "-O3", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  r = hiprtcCompileProgram(prog, 6, opts);
  size_t logn = 0;
  hiprtcGetProgramLogSize(prog, &logn);
  std::string logs(logn, '\0');
  if (logn > 1) hiprtcGetProgramLog(prog, &logs[0]);
  if (r != HIPRTC_SUCCESS) {
    if (log) {
      *log = (char *)malloc(logs.size() + 1);
      memcpy(*log, logs.c_str(), logs.size() + 1);
    }
    hiprtcDestroyProgram(&prog);
    return fail(CTHIP_E_COMPILE, "cthip_compile: hiprtc (%s %s) failed: %s\n%s", archopt.c_str(), "-O3",
                hiprtcGetErrorString(r), logs.c_str());
  }
  size_t n = 0;
  hiprtcGetCodeSize(prog, &n);
  char *buf = (char *)malloc(n);
  hiprtcGetCode(prog, buf);
  hiprtcDestroyProgram(&prog);
  *code = buf;
  *code_size = n;
  return 0;
}

void cthip_release(void *p) { free(p); }

int cthip_module_load(void **module, const void *code) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(module != nullptr && code != nullptr);
  hipModule_t m;
  CTHIP_CHECK(hipModuleLoadData(&m, code));
  *module = (void *)m;
  return 0;
}

int cthip_module_unload(void *module) {
  CTHIP_REQUIRE_INIT();
  if (!module) return 0;
  CTHIP_CHECK(hipStreamSynchronize(state().stream));
  CTHIP_CHECK(hipModuleUnload((hipModule_t)module));
  return 0;
}

int cthip_get_function(void **fn, void *module, const char *name) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(fn != nullptr && module != nullptr && name != nullptr);
  hipFunction_t f;
  hipError_t e = hipModuleGetFunction(&f, (hipModule_t)module, name);
  if (e != hipSuccess) return fail((int)e, "cthip_get_function: no kernel named '%s' in module: %s", name, hipGetErrorString(e));
  *fn = (void *)f;
  return 0;
}

int cthip_launch(void *fn, const unsigned grid[3], const unsigned block[3], unsigned lds_bytes, void **args,
                 int nargs) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(fn != nullptr && grid != nullptr && block != nullptr && nargs >= 0 && (nargs == 0 || args != nullptr));
  if ((size_t)block[0] * block[1] * block[2] == 0 || (size_t)block[0] * block[1] * block[2] > 1024)
    return fail(CTHIP_E_BAD_ARG, "cthip_launch: block %ux%ux%u is outside 1..1024 threads", block[0], block[1], block[2]);
  if ((size_t)grid[0] * grid[1] * grid[2] == 0) return 0;  // empty iteration space: nothing to do
  if (lds_bytes > 160 * 1024) return fail(CTHIP_E_BAD_ARG, "cthip_launch: %u bytes of LDS exceed 160 KiB", lds_bytes);
  CTHIP_CHECK(hipModuleLaunchKernel((hipFunction_t)fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                    lds_bytes, state().stream, args, nullptr));
  return 0;
}

}  // extern "C"

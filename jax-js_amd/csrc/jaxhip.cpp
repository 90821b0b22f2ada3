// jaxhip.cpp -- the C-ABI runtime declared in include/jaxhip.h.
//
// Thin by design: hipMalloc / hipMemcpyAsync / hiprtc / hipModuleLaunchKernel on one in-order
// stream.  Slots, reference counting, the kernel cache and code generation live in the host-side
// HipBackend; see the header for which reference interface each entry point stands in for.

#include "jaxhip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

// Scratch memory of `jh_launch_static_scratch`: one array per GPU, inside the library's own code object, so the entry
// point never allocates.  In host code the array's name is only a stand-in: the device address is looked up once
// per device (hipGetSymbolAddress in jh_init) and that pointer is what kernels receive.
#define JH_STATIC_SCRATCH_BYTES (32u << 20)
static __device__ __align__(256) unsigned char jh_static_scratch[JH_STATIC_SCRATCH_BYTES];

namespace {

thread_local std::string g_last_error;

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices] = {};  // device address of jh_static_scratch on each GPU this process has initialised

// Large reads from the device into pageable host memory go through two pinned buffers: the CPU drains one while the
// DMA engine fills the other (134 MB: 26-27 GB/s against 17 GB/s for a direct hipMemcpy into pageable memory; uploads
// are left to the runtime, whose own pageable path measured 29 GB/s against 27 through these buffers).
constexpr size_t kStageChunk = 8u << 20;    // bytes per pinned buffer
constexpr size_t kStageFrom = 1u << 20;     // smaller reads are left to the runtime

struct Runtime {
  bool ready = false;
  int device = -1;
  hipStream_t stream = nullptr;
  void *stage[2] = {nullptr, nullptr};      // pinned staging buffers, allocated at the first large read
  hipEvent_t stage_ev[2] = {nullptr, nullptr};
  bool stage_tried = false;
};
Runtime g_rt;

int fail(int code, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code ? code : -1;
}

#define JH_HIP(expr)                                                                      \
  do {                                                                                    \
    hipError_t e_ = (expr);                                                               \
    if (e_ != hipSuccess) return fail((int)e_, "%s failed: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

#define JH_NEED_INIT()                                                  \
  do {                                                                  \
    if (!g_rt.ready) return fail(-2, "jh_init has not been called");    \
  } while (0)

// The staging buffers, or false when pinned memory cannot be had (the caller then copies directly).
bool stage_ready() {
  if (g_rt.stage_tried) return g_rt.stage[0] != nullptr;
  g_rt.stage_tried = true;
  void *b0 = nullptr, *b1 = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipHostMalloc(&b0, kStageChunk, hipHostMallocDefault) == hipSuccess && hipHostMalloc(&b1, kStageChunk, hipHostMallocDefault) == hipSuccess &&
      hipEventCreateWithFlags(&e0, hipEventDisableTiming) == hipSuccess && hipEventCreateWithFlags(&e1, hipEventDisableTiming) == hipSuccess) {
    g_rt.stage[0] = b0, g_rt.stage[1] = b1, g_rt.stage_ev[0] = e0, g_rt.stage_ev[1] = e1;
    return true;
  }
  if (b0) (void)hipHostFree(b0);
  if (b1) (void)hipHostFree(b1);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipGetLastError();
  return false;
}

void stage_release() {
  for (int b = 0; b < 2; ++b) {
    if (g_rt.stage[b]) (void)hipHostFree(g_rt.stage[b]);
    if (g_rt.stage_ev[b]) (void)hipEventDestroy(g_rt.stage_ev[b]);
  }
}

}  // namespace

extern "C" {

int jh_abi_version(void) { return 2; }

const char *jh_last_error(void) { return g_last_error.c_str(); }

int jh_init(int device) {
  if (g_rt.ready) {
    if (g_rt.device == device) return 0;
    return fail(-3, "runtime already initialised on device %d", g_rt.device);
  }
  int count = 0;
  JH_HIP(hipGetDeviceCount(&count));
  if (device < 0 || device >= count) return fail(-4, "device %d out of range (%d visible)", device, count);
  JH_HIP(hipSetDevice(device));
  // Default priority on purpose: work on streams of different priorities has hung on this pool.
  JH_HIP(hipStreamCreateWithFlags(&g_rt.stream, hipStreamNonBlocking));
  if (device < kMaxDevices && !g_scratch_ptr[device]) {
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(jh_static_scratch));  // this device's copy of the array
    if (e != hipSuccess || !p) {
      (void)hipStreamDestroy(g_rt.stream);
      g_rt.stream = nullptr;
      return fail((int)e ? (int)e : -9, "hipGetSymbolAddress(jh_static_scratch) failed: %s", hipGetErrorString(e));
    }
    g_scratch_ptr[device] = p;
  }
  g_rt.device = device;
  g_rt.ready = true;
  return 0;
}

int jh_shutdown(void) {
  if (!g_rt.ready) return 0;
  JH_HIP(hipStreamSynchronize(g_rt.stream));
  stage_release();
  JH_HIP(hipStreamDestroy(g_rt.stream));
  g_rt = Runtime();
  return 0;
}

int jh_get_device_info(jh_device_info *out) {
  JH_NEED_INIT();
  if (!out) return fail(-5, "null output");
  hipDeviceProp_t p;
  JH_HIP(hipGetDeviceProperties(&p, g_rt.device));
  memset(out, 0, sizeof(*out));
  snprintf(out->name, sizeof(out->name), "%s", p.name);
  snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
  out->compute_units = p.multiProcessorCount;
  out->wavefront_size = p.warpSize;
  out->max_threads_per_block = p.maxThreadsPerBlock;
  out->lds_bytes_per_block = (int32_t)p.sharedMemPerBlock;
  out->total_mem_bytes = (int64_t)p.totalGlobalMem;
  out->clock_khz = p.clockRate;
  out->l2_bytes = p.l2CacheSize;
  return 0;
}

int jh_malloc(size_t bytes, jh_devptr *out) {
  JH_NEED_INIT();
  if (!out) return fail(-5, "null output");
  *out = nullptr;
  if (bytes == 0) return 0;
  JH_HIP(hipMalloc(out, bytes));
  return 0;
}

int jh_free(jh_devptr ptr) {
  JH_NEED_INIT();
  if (!ptr) return 0;
  // hipFree waits for the device, so a buffer still read by a queued kernel is safe to release.
  JH_HIP(hipFree(ptr));
  return 0;
}

int jh_memcpy_h2d(jh_devptr dst, const void *src, size_t bytes) {
  JH_NEED_INIT();
  if (bytes == 0) return 0;
  if (!dst || !src) return fail(-5, "null pointer in h2d copy");
  JH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_rt.stream));
  // Pageable source memory: make sure the runtime is done reading it before the caller reuses it.
  JH_HIP(hipStreamSynchronize(g_rt.stream));
  return 0;
}

int jh_memcpy_d2h(void *dst, jh_devptr src, size_t offset, size_t bytes) {
  JH_NEED_INIT();
  if (bytes == 0) {
    JH_HIP(hipStreamSynchronize(g_rt.stream));
    return 0;
  }
  if (!dst || !src) return fail(-5, "null pointer in d2h copy");
  if (bytes >= kStageFrom && stage_ready()) {
    // The device fills pinned buffer (i + 1) % 2 while the CPU drains buffer i % 2.
    const size_t chunks = (bytes + kStageChunk - 1) / kStageChunk;
    auto issue = [&](size_t i) -> hipError_t {
      const size_t off = i * kStageChunk, n = bytes - off < kStageChunk ? bytes - off : kStageChunk;
      hipError_t e = hipMemcpyAsync(g_rt.stage[i & 1], (const char *)src + offset + off, n, hipMemcpyDeviceToHost, g_rt.stream);
      return e != hipSuccess ? e : hipEventRecord(g_rt.stage_ev[i & 1], g_rt.stream);
    };
    JH_HIP(issue(0));
    for (size_t i = 0; i < chunks; ++i) {
      if (i + 1 < chunks) JH_HIP(issue(i + 1));
      const size_t off = i * kStageChunk, n = bytes - off < kStageChunk ? bytes - off : kStageChunk;
      JH_HIP(hipEventSynchronize(g_rt.stage_ev[i & 1]));
      memcpy((char *)dst + off, g_rt.stage[i & 1], n);
    }
    return 0;
  }
  JH_HIP(hipMemcpyAsync(dst, (const char *)src + offset, bytes, hipMemcpyDeviceToHost, g_rt.stream));
  JH_HIP(hipStreamSynchronize(g_rt.stream));
  return 0;
}

int jh_memcpy_d2h_async(void *dst, jh_devptr src, size_t offset, size_t bytes, jh_event *done) {
  JH_NEED_INIT();
  if (!done) return fail(-5, "null event output");
  if (bytes != 0) {
    if (!dst || !src) return fail(-5, "null pointer in d2h copy");
    JH_HIP(hipMemcpyAsync(dst, (const char *)src + offset, bytes, hipMemcpyDeviceToHost, g_rt.stream));
  }
  hipEvent_t ev;
  JH_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
  hipError_t e = hipEventRecord(ev, g_rt.stream);
  if (e != hipSuccess) {
    (void)hipEventDestroy(ev);
    return fail((int)e, "hipEventRecord failed: %s", hipGetErrorString(e));
  }
  *done = (jh_event)ev;
  return 0;
}

int jh_memcpy_d2d(jh_devptr dst, jh_devptr src, size_t bytes) {
  JH_NEED_INIT();
  if (bytes == 0) return 0;
  if (!dst || !src) return fail(-5, "null pointer in d2d copy");
  JH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_rt.stream));
  return 0;
}

int jh_host_alloc(size_t bytes, void **out) {
  JH_NEED_INIT();
  if (!out) return fail(-5, "null output");
  *out = nullptr;
  if (bytes == 0) return 0;
  JH_HIP(hipHostMalloc(out, bytes, hipHostMallocDefault));
  return 0;
}

int jh_host_free(void *ptr) {
  // No JH_NEED_INIT: a garbage collector may hand pinned memory back after jh_shutdown; hipHostFree needs no stream.
  if (!ptr) return 0;
  JH_HIP(hipHostFree(ptr));
  return 0;
}

int jh_compile(const char *source, const char *name, const char *const *options, int num_options, void **code,
               size_t *code_size, char *log, size_t log_size) {
  if (!source || !code || !code_size) return fail(-5, "null argument to jh_compile");
  *code = nullptr;
  *code_size = 0;
  if (log && log_size) log[0] = '\0';
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, name ? name : "kernel.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return fail((int)r, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
  // Options the source asks for itself: leading lines of the form "// hiprtc-option: <option>", honoured for the
  // options on a fixed list (the generator marks float16 kernels that the SLP vectorizer makes the compiler abort on).
  std::vector<std::string> asked;
  {
    static const char kMark[] = "// hiprtc-option: ";
    static const char *const kAllowed[] = {"-fno-slp-vectorize"};
    const char *line = source;
    while (strncmp(line, kMark, sizeof(kMark) - 1) == 0) {
      const char *begin = line + sizeof(kMark) - 1;
      const char *end = strchr(begin, '\n');
      std::string opt = end ? std::string(begin, end) : std::string(begin);
      while (!opt.empty() && (opt.back() == ' ' || opt.back() == '\r')) opt.pop_back();
      bool ok = false;
      for (const char *a : kAllowed) ok = ok || opt == a;
      if (!ok) {
        hiprtcDestroyProgram(&prog);
        return fail(-5, "the source asks for a compiler option that is not on the list: %s", opt.c_str());
      }
      bool present = false;
      for (int i = 0; i < num_options; ++i) present = present || (options[i] && opt == options[i]);
      if (!present) asked.push_back(opt);
      if (!end) break;
      line = end + 1;
    }
  }
  std::vector<const char *> all_options(options, options + (options ? num_options : 0));
  for (const std::string &o : asked) all_options.push_back(o.c_str());
  r = hiprtcCompileProgram(prog, (int)all_options.size(), all_options.data());
  size_t n = 0;
  if (hiprtcGetProgramLogSize(prog, &n) == HIPRTC_SUCCESS && n > 1) {
    std::string text(n, '\0');
    if (hiprtcGetProgramLog(prog, &text[0]) == HIPRTC_SUCCESS) {
      if (log && log_size) snprintf(log, log_size, "%s", text.c_str());
      if (r != HIPRTC_SUCCESS) g_last_error = text;
    }
  }
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    if (g_last_error.empty()) g_last_error = hiprtcGetErrorString(r);
    return (int)r;
  }
  size_t sz = 0;
  r = hiprtcGetCodeSize(prog, &sz);
  if (r != HIPRTC_SUCCESS || sz == 0) {
    hiprtcDestroyProgram(&prog);
    return fail((int)r ? (int)r : -6, "hiprtcGetCodeSize: %s", hiprtcGetErrorString(r));
  }
  void *buf = malloc(sz);
  if (!buf) {
    hiprtcDestroyProgram(&prog);
    return fail(-7, "out of host memory for %zu byte code object", sz);
  }
  r = hiprtcGetCode(prog, (char *)buf);
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    free(buf);
    return fail((int)r, "hiprtcGetCode: %s", hiprtcGetErrorString(r));
  }
  *code = buf;
  *code_size = sz;
  return 0;
}

void jh_code_free(void *code) { free(code); }

int jh_compiler_version(int *major, int *minor) {
  if (!major || !minor) return fail(-5, "null output");
  hiprtcResult r = hiprtcVersion(major, minor);
  if (r != HIPRTC_SUCCESS) return fail((int)r, "hiprtcVersion: %s", hiprtcGetErrorString(r));
  return 0;
}

int jh_module_load(const void *code, size_t code_size, jh_module *out) {
  JH_NEED_INIT();
  if (!code || !code_size || !out) return fail(-5, "null argument to jh_module_load");
  hipModule_t m;
  JH_HIP(hipModuleLoadData(&m, code));
  *out = (jh_module)m;
  return 0;
}

int jh_module_unload(jh_module module) {
  JH_NEED_INIT();
  if (!module) return 0;
  JH_HIP(hipModuleUnload((hipModule_t)module));
  return 0;
}

int jh_module_function(jh_module module, const char *kernel_name, jh_function *out) {
  JH_NEED_INIT();
  if (!module || !kernel_name || !out) return fail(-5, "null argument to jh_module_function");
  hipFunction_t f;
  JH_HIP(hipModuleGetFunction(&f, (hipModule_t)module, kernel_name));
  *out = (jh_function)f;
  return 0;
}

int jh_launch(jh_function fn, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz,
              uint32_t shared_bytes, void **args) {
  JH_NEED_INIT();
  if (!fn) return fail(-5, "null kernel");
  if (gx == 0 || gy == 0 || gz == 0) return 0;  // empty grid: nothing to do
  if (bx == 0 || by == 0 || bz == 0 || (uint64_t)bx * by * bz > 1024)
    return fail(-8, "invalid block %ux%ux%u", bx, by, bz);
  JH_HIP(hipModuleLaunchKernel((hipFunction_t)fn, gx, gy, gz, bx, by, bz, shared_bytes, g_rt.stream, args, nullptr));
  return 0;
}

int jh_static_scratch_bytes(size_t *bytes) {
  if (!bytes) return fail(-5, "null output");
  *bytes = JH_STATIC_SCRATCH_BYTES;
  return 0;
}

int jh_launch_static_scratch(jh_function fn, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz,
                             uint32_t shared_bytes, void **args, uint32_t scratch_arg, size_t scratch_bytes) {
  JH_NEED_INIT();
  if (!fn || !args) return fail(-5, "null kernel or argument list");
  if (scratch_bytes > JH_STATIC_SCRATCH_BYTES)
    return fail(-10, "kernel needs %zu bytes of scratch, the static scratch buffer holds %u", scratch_bytes,
                (unsigned)JH_STATIC_SCRATCH_BYTES);
  if (g_rt.device >= kMaxDevices || !g_scratch_ptr[g_rt.device]) return fail(-9, "no static scratch on device %d", g_rt.device);
  if (!args[scratch_arg]) return fail(-5, "argument %u has no cell to receive the scratch address", scratch_arg);
  // The kernel takes the looked-up device address, never the array's name.
  *(void **)args[scratch_arg] = g_scratch_ptr[g_rt.device];
  return jh_launch(fn, gx, gy, gz, bx, by, bz, shared_bytes, args);
}

int jh_launch_repeat(jh_function fn, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz,
                     uint32_t shared_bytes, void **args, int count) {
  for (int i = 0; i < count; i++) {
    int rc = jh_launch(fn, gx, gy, gz, bx, by, bz, shared_bytes, args);
    if (rc) return rc;
  }
  return 0;
}

int jh_graph_begin(void) {
  JH_NEED_INIT();
  JH_HIP(hipStreamBeginCapture(g_rt.stream, hipStreamCaptureModeThreadLocal));
  return 0;
}

int jh_graph_end(jh_graph *out) {
  JH_NEED_INIT();
  if (!out) return fail(-5, "null output");
  hipGraph_t graph = nullptr;
  JH_HIP(hipStreamEndCapture(g_rt.stream, &graph));
  hipGraphExec_t exec = nullptr;
  hipError_t err = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (err != hipSuccess) return fail((int)err, "hipGraphInstantiate failed: %s", hipGetErrorString(err));
  *out = (jh_graph)exec;
  return 0;
}

int jh_graph_launch(jh_graph graph) {
  JH_NEED_INIT();
  if (!graph) return fail(-5, "null graph");
  JH_HIP(hipGraphLaunch((hipGraphExec_t)graph, g_rt.stream));
  return 0;
}

int jh_graph_destroy(jh_graph graph) {
  JH_NEED_INIT();
  if (!graph) return 0;
  JH_HIP(hipGraphExecDestroy((hipGraphExec_t)graph));
  return 0;
}

int jh_sync(void) {
  JH_NEED_INIT();
  JH_HIP(hipStreamSynchronize(g_rt.stream));
  return 0;
}

int jh_event_create(jh_event *out) {
  JH_NEED_INIT();
  if (!out) return fail(-5, "null output");
  hipEvent_t ev;
  JH_HIP(hipEventCreate(&ev));
  *out = (jh_event)ev;
  return 0;
}

int jh_event_record(jh_event ev) {
  JH_NEED_INIT();
  if (!ev) return fail(-5, "null event");
  JH_HIP(hipEventRecord((hipEvent_t)ev, g_rt.stream));
  return 0;
}

int jh_event_query(jh_event ev, int *done) {
  JH_NEED_INIT();
  if (!ev || !done) return fail(-5, "null argument");
  hipError_t e = hipEventQuery((hipEvent_t)ev);
  if (e == hipSuccess) {
    *done = 1;
    return 0;
  }
  if (e == hipErrorNotReady) {
    *done = 0;
    return 0;
  }
  return fail((int)e, "hipEventQuery failed: %s", hipGetErrorString(e));
}

int jh_event_sync(jh_event ev) {
  JH_NEED_INIT();
  if (!ev) return fail(-5, "null event");
  JH_HIP(hipEventSynchronize((hipEvent_t)ev));
  return 0;
}

int jh_event_elapsed_ms(jh_event start, jh_event stop, float *ms) {
  JH_NEED_INIT();
  if (!start || !stop || !ms) return fail(-5, "null argument");
  JH_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return 0;
}

int jh_event_destroy(jh_event ev) {
  JH_NEED_INIT();
  if (!ev) return 0;
  JH_HIP(hipEventDestroy((hipEvent_t)ev));
  return 0;
}

}  // extern "C"

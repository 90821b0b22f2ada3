// N-API addon over the C ABI of libjaxhip (include/jaxhip.h): what a JavaScript `HipBackend` binds.
//
// One export per C entry point; device addresses and handles cross as BigInt, host memory as
// Uint8Array/Buffer.  Every export throws a JavaScript Error carrying jh_last_error() when the C call
// reports a non-zero status, which is how the Backend interface signals failure (exceptions, never codes;
// src/backend.ts:222-240).  N-API is ABI-stable, so one build serves every Node version from 12.17 on
// (BigInt support, N-API 6).
#include <node_api.h>

#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "jaxhip.h"

namespace {

#define NAPI_OK(call)                                                  \
  do {                                                                 \
    if ((call) != napi_ok) {                                           \
      napi_throw_error(env, nullptr, "jaxhip: bad argument (" #call ")"); \
      return nullptr;                                                  \
    }                                                                  \
  } while (0)

#define JH_OK(call)                                        \
  do {                                                     \
    if ((call) != 0) {                                     \
      napi_throw_error(env, nullptr, jh_last_error());     \
      return nullptr;                                      \
    }                                                      \
  } while (0)

struct Args {
  napi_env env;
  size_t argc = 8;
  napi_value argv[8];
  bool ok;
  Args(napi_env e, napi_callback_info info) : env(e) {
    ok = napi_get_cb_info(env, info, &argc, argv, nullptr, nullptr) == napi_ok;
  }
};

bool get_u64(napi_env env, napi_value v, uint64_t* out) {
  napi_valuetype t;
  if (napi_typeof(env, v, &t) != napi_ok) return false;
  if (t == napi_bigint) {
    bool lossless = false;
    return napi_get_value_bigint_uint64(env, v, out, &lossless) == napi_ok;
  }
  if (t == napi_number) {
    double d;
    if (napi_get_value_double(env, v, &d) != napi_ok || d < 0) return false;
    *out = (uint64_t)d;
    return true;
  }
  return false;
}

napi_value make_u64(napi_env env, uint64_t v) {
  napi_value out;
  napi_create_bigint_uint64(env, v, &out);
  return out;
}

bool get_bytes(napi_env env, napi_value v, void** data, size_t* len) {
  bool is_ta = false;
  if (napi_is_typedarray(env, v, &is_ta) == napi_ok && is_ta) {
    napi_typedarray_type type;
    size_t n, off;
    napi_value ab;
    if (napi_get_typedarray_info(env, v, &type, &n, data, &ab, &off) != napi_ok) return false;
    size_t width = 1;
    switch (type) {
      case napi_int16_array: case napi_uint16_array: width = 2; break;
      case napi_int32_array: case napi_uint32_array: case napi_float32_array: width = 4; break;
      case napi_float64_array: case napi_bigint64_array: case napi_biguint64_array: width = 8; break;
      default: width = 1;
    }
    *len = n * width;
    return true;
  }
  bool is_buf = false;
  if (napi_is_buffer(env, v, &is_buf) == napi_ok && is_buf) return napi_get_buffer_info(env, v, data, len) == napi_ok;
  return false;
}

bool get_string(napi_env env, napi_value v, std::string* out) {
  size_t n = 0;
  if (napi_get_value_string_utf8(env, v, nullptr, 0, &n) != napi_ok) return false;
  out->resize(n);
  return napi_get_value_string_utf8(env, v, &(*out)[0], n + 1, &n) == napi_ok;
}

napi_value Init(napi_env env, napi_callback_info info) {
  Args a(env, info);
  int32_t device = 0;
  if (a.argc >= 1) NAPI_OK(napi_get_value_int32(env, a.argv[0], &device));
  JH_OK(jh_init(device));
  return nullptr;
}

napi_value Shutdown(napi_env env, napi_callback_info) {
  JH_OK(jh_shutdown());
  return nullptr;
}

napi_value DeviceInfo(napi_env env, napi_callback_info) {
  jh_device_info d;
  JH_OK(jh_get_device_info(&d));
  napi_value o, v;
  napi_create_object(env, &o);
  napi_create_string_utf8(env, d.name, NAPI_AUTO_LENGTH, &v); napi_set_named_property(env, o, "name", v);
  napi_create_string_utf8(env, d.arch, NAPI_AUTO_LENGTH, &v); napi_set_named_property(env, o, "arch", v);
  napi_create_int32(env, d.compute_units, &v); napi_set_named_property(env, o, "computeUnits", v);
  napi_create_int32(env, d.wavefront_size, &v); napi_set_named_property(env, o, "wavefrontSize", v);
  napi_create_int32(env, d.lds_bytes_per_block, &v); napi_set_named_property(env, o, "ldsBytesPerBlock", v);
  napi_create_double(env, (double)d.total_mem_bytes, &v); napi_set_named_property(env, o, "totalMemBytes", v);
  return o;
}

napi_value Malloc(napi_env env, napi_callback_info info) {  // malloc(bytes) -> BigInt device address
  Args a(env, info);
  uint64_t bytes;
  if (a.argc < 1 || !get_u64(env, a.argv[0], &bytes)) { napi_throw_type_error(env, nullptr, "malloc(bytes)"); return nullptr; }
  jh_devptr p = nullptr;
  JH_OK(jh_malloc((size_t)bytes, &p));
  return make_u64(env, (uint64_t)(uintptr_t)p);
}

napi_value Free(napi_env env, napi_callback_info info) {
  Args a(env, info);
  uint64_t p;
  if (a.argc < 1 || !get_u64(env, a.argv[0], &p)) { napi_throw_type_error(env, nullptr, "free(ptr)"); return nullptr; }
  JH_OK(jh_free((jh_devptr)(uintptr_t)p));
  return nullptr;
}

napi_value H2D(napi_env env, napi_callback_info info) {  // h2d(dst, bytes: Uint8Array)
  Args a(env, info);
  uint64_t dst;
  void* data; size_t len;
  if (a.argc < 2 || !get_u64(env, a.argv[0], &dst) || !get_bytes(env, a.argv[1], &data, &len)) {
    napi_throw_type_error(env, nullptr, "h2d(dst, typedArray)"); return nullptr;
  }
  if (len) JH_OK(jh_memcpy_h2d((jh_devptr)(uintptr_t)dst, data, len));
  return nullptr;
}

napi_value D2H(napi_env env, napi_callback_info info) {  // d2h(src, offset, bytes) -> Uint8Array (ordered after prior launches)
  Args a(env, info);
  uint64_t src, off, bytes;
  if (a.argc < 3 || !get_u64(env, a.argv[0], &src) || !get_u64(env, a.argv[1], &off) || !get_u64(env, a.argv[2], &bytes)) {
    napi_throw_type_error(env, nullptr, "d2h(src, offset, bytes)"); return nullptr;
  }
  napi_value ab, out;
  void* data = nullptr;
  NAPI_OK(napi_create_arraybuffer(env, (size_t)bytes, &data, &ab));
  if (bytes) JH_OK(jh_memcpy_d2h(data, (jh_devptr)(uintptr_t)src, (size_t)off, (size_t)bytes));
  else JH_OK(jh_sync());  // read(slot, 0, 0) is the caller's completion fence
  NAPI_OK(napi_create_typedarray(env, napi_uint8_array, (size_t)bytes, ab, 0, &out));
  return out;
}

napi_value D2D(napi_env env, napi_callback_info info) {  // d2d(dst, src, bytes): copy on the stream, in dispatch order
  Args a(env, info);
  uint64_t dst, src, bytes;
  if (a.argc < 3 || !get_u64(env, a.argv[0], &dst) || !get_u64(env, a.argv[1], &src) || !get_u64(env, a.argv[2], &bytes)) {
    napi_throw_type_error(env, nullptr, "d2d(dst, src, bytes)"); return nullptr;
  }
  if (bytes) JH_OK(jh_memcpy_d2d((jh_devptr)(uintptr_t)dst, (jh_devptr)(uintptr_t)src, (size_t)bytes));
  return nullptr;
}

// Runs when the collector drops the buffer, possibly after shutdown() or at process exit: jh_host_free needs no
// initialised runtime and its status is ignored here (there is nobody to report it to).
void free_pinned(napi_env, void* data, void*) {  // finalizer of the array buffers d2hAsync hands out
  if (data) (void)jh_host_free(data);
}

// d2hAsync(src, offset, bytes) -> {event: BigInt, data: Uint8Array}.  The copy into pinned host memory is queued behind
// every earlier launch and the call returns at once; `data` holds the bytes once eventQuery(event) reports true.  The
// pinned memory belongs to the returned array buffer and is released when that is collected.
napi_value D2HAsync(napi_env env, napi_callback_info info) {
  Args a(env, info);
  uint64_t src, off, bytes;
  if (a.argc < 3 || !get_u64(env, a.argv[0], &src) || !get_u64(env, a.argv[1], &off) || !get_u64(env, a.argv[2], &bytes)) {
    napi_throw_type_error(env, nullptr, "d2hAsync(src, offset, bytes)"); return nullptr;
  }
  void* host = nullptr;
  if (bytes) JH_OK(jh_host_alloc((size_t)bytes, &host));
  jh_event ev = nullptr;
  if (jh_memcpy_d2h_async(host, (jh_devptr)(uintptr_t)src, (size_t)off, (size_t)bytes, &ev) != 0) {
    if (host) (void)jh_host_free(host);
    napi_throw_error(env, nullptr, jh_last_error());
    return nullptr;
  }
  napi_value ab, arr, out;
  napi_status st = bytes ? napi_create_external_arraybuffer(env, host, (size_t)bytes, free_pinned, nullptr, &ab)
                         : napi_create_arraybuffer(env, 0, &host, &ab);
  if (st != napi_ok) {
    (void)jh_event_sync(ev); (void)jh_event_destroy(ev);
    if (bytes && host) (void)jh_host_free(host);
    napi_throw_error(env, nullptr, "jaxhip: cannot wrap pinned memory in an ArrayBuffer");
    return nullptr;
  }
  NAPI_OK(napi_create_typedarray(env, napi_uint8_array, (size_t)bytes, ab, 0, &arr));
  NAPI_OK(napi_create_object(env, &out));
  NAPI_OK(napi_set_named_property(env, out, "event", make_u64(env, (uint64_t)(uintptr_t)ev)));
  NAPI_OK(napi_set_named_property(env, out, "data", arr));
  return out;
}

napi_value CompilerVersion(napi_env env, napi_callback_info) {  // "major.minor" of hiprtc (part of a code-object cache key)
  int major = 0, minor = 0;
  JH_OK(jh_compiler_version(&major, &minor));
  napi_value out;
  napi_create_string_utf8(env, (std::to_string(major) + "." + std::to_string(minor)).c_str(), NAPI_AUTO_LENGTH, &out);
  return out;
}

napi_value Compile(napi_env env, napi_callback_info info) {  // compile(source, name, options: string[]) -> Buffer
  Args a(env, info);
  std::string source, name;
  if (a.argc < 2 || !get_string(env, a.argv[0], &source) || !get_string(env, a.argv[1], &name)) {
    napi_throw_type_error(env, nullptr, "compile(source, name, options)"); return nullptr;
  }
  std::vector<std::string> opts;
  if (a.argc >= 3) {
    uint32_t n = 0;
    NAPI_OK(napi_get_array_length(env, a.argv[2], &n));
    for (uint32_t i = 0; i < n; ++i) {
      napi_value e; std::string s;
      NAPI_OK(napi_get_element(env, a.argv[2], i, &e));
      if (!get_string(env, e, &s)) { napi_throw_type_error(env, nullptr, "options must be strings"); return nullptr; }
      opts.push_back(s);
    }
  }
  std::vector<const char*> optv;
  for (auto& s : opts) optv.push_back(s.c_str());
  void* code = nullptr; size_t size = 0;
  std::vector<char> log(1 << 16, 0);
  if (jh_compile(source.c_str(), name.c_str(), optv.data(), (int)optv.size(), &code, &size, log.data(), log.size()) != 0) {
    std::string msg = std::string(jh_last_error()) + "\n" + log.data();
    napi_throw_error(env, nullptr, msg.c_str());
    return nullptr;
  }
  napi_value buf; void* dst = nullptr;
  napi_status st = napi_create_buffer_copy(env, size, code, &dst, &buf);
  jh_code_free(code);
  NAPI_OK(st);
  return buf;
}

napi_value ModuleLoad(napi_env env, napi_callback_info info) {  // moduleLoad(code: Buffer) -> BigInt
  Args a(env, info);
  void* data; size_t len;
  if (a.argc < 1 || !get_bytes(env, a.argv[0], &data, &len)) { napi_throw_type_error(env, nullptr, "moduleLoad(code)"); return nullptr; }
  jh_module m = nullptr;
  JH_OK(jh_module_load(data, len, &m));
  return make_u64(env, (uint64_t)(uintptr_t)m);
}

napi_value ModuleUnload(napi_env env, napi_callback_info info) {
  Args a(env, info);
  uint64_t m;
  if (a.argc < 1 || !get_u64(env, a.argv[0], &m)) { napi_throw_type_error(env, nullptr, "moduleUnload(module)"); return nullptr; }
  JH_OK(jh_module_unload((jh_module)(uintptr_t)m));
  return nullptr;
}

napi_value ModuleFunction(napi_env env, napi_callback_info info) {  // moduleFunction(module, name) -> BigInt
  Args a(env, info);
  uint64_t m; std::string name;
  if (a.argc < 2 || !get_u64(env, a.argv[0], &m) || !get_string(env, a.argv[1], &name)) {
    napi_throw_type_error(env, nullptr, "moduleFunction(module, name)"); return nullptr;
  }
  jh_function f = nullptr;
  JH_OK(jh_module_function((jh_module)(uintptr_t)m, name.c_str(), &f));
  return make_u64(env, (uint64_t)(uintptr_t)f);
}

bool get_dim3(napi_env env, napi_value v, uint32_t out[3]) {
  uint32_t n = 0;
  if (napi_get_array_length(env, v, &n) != napi_ok || n != 3) return false;
  for (uint32_t i = 0; i < 3; ++i) {
    napi_value e;
    if (napi_get_element(env, v, i, &e) != napi_ok || napi_get_value_uint32(env, e, &out[i]) != napi_ok) return false;
  }
  return true;
}

napi_value Launch(napi_env env, napi_callback_info info) {  // launch(fn, [gx,gy,gz], [bx,by,bz], sharedBytes, ptrs: BigInt[], repeat?)
  Args a(env, info);
  uint64_t fn; uint32_t grid[3], block[3], shared = 0, nargs = 0, repeat = 1;
  if (a.argc < 5 || !get_u64(env, a.argv[0], &fn) || !get_dim3(env, a.argv[1], grid) || !get_dim3(env, a.argv[2], block) ||
      napi_get_value_uint32(env, a.argv[3], &shared) != napi_ok || napi_get_array_length(env, a.argv[4], &nargs) != napi_ok) {
    napi_throw_type_error(env, nullptr, "launch(fn, grid[3], block[3], sharedBytes, pointers[])"); return nullptr;
  }
  if (a.argc >= 6) NAPI_OK(napi_get_value_uint32(env, a.argv[5], &repeat));
  std::vector<uint64_t> vals(nargs);
  std::vector<void*> argv(nargs);
  for (uint32_t i = 0; i < nargs; ++i) {
    napi_value e;
    NAPI_OK(napi_get_element(env, a.argv[4], i, &e));
    if (!get_u64(env, e, &vals[i])) { napi_throw_type_error(env, nullptr, "kernel arguments must be BigInt device addresses"); return nullptr; }
    argv[i] = &vals[i];
  }
  JH_OK(jh_launch_repeat((jh_function)(uintptr_t)fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], shared,
                         argv.data(), (int)repeat));
  return nullptr;
}

napi_value Sync(napi_env env, napi_callback_info) {
  JH_OK(jh_sync());
  return nullptr;
}

napi_value EventCreate(napi_env env, napi_callback_info) {
  jh_event e = nullptr;
  JH_OK(jh_event_create(&e));
  return make_u64(env, (uint64_t)(uintptr_t)e);
}

napi_value EventRecord(napi_env env, napi_callback_info info) {
  Args a(env, info);
  uint64_t e;
  if (a.argc < 1 || !get_u64(env, a.argv[0], &e)) { napi_throw_type_error(env, nullptr, "eventRecord(event)"); return nullptr; }
  JH_OK(jh_event_record((jh_event)(uintptr_t)e));
  return nullptr;
}

napi_value EventQuery(napi_env env, napi_callback_info info) {  // non-blocking: true once the event has passed
  Args a(env, info);
  uint64_t e; int done = 0;
  if (a.argc < 1 || !get_u64(env, a.argv[0], &e)) { napi_throw_type_error(env, nullptr, "eventQuery(event)"); return nullptr; }
  JH_OK(jh_event_query((jh_event)(uintptr_t)e, &done));
  napi_value out;
  napi_get_boolean(env, done != 0, &out);
  return out;
}

napi_value EventElapsed(napi_env env, napi_callback_info info) {
  Args a(env, info);
  uint64_t e0, e1; float ms = 0;
  if (a.argc < 2 || !get_u64(env, a.argv[0], &e0) || !get_u64(env, a.argv[1], &e1)) {
    napi_throw_type_error(env, nullptr, "eventElapsedMs(start, stop)"); return nullptr;
  }
  JH_OK(jh_event_sync((jh_event)(uintptr_t)e1));
  JH_OK(jh_event_elapsed_ms((jh_event)(uintptr_t)e0, (jh_event)(uintptr_t)e1, &ms));
  napi_value out;
  napi_create_double(env, ms, &out);
  return out;
}

napi_value EventDestroy(napi_env env, napi_callback_info info) {
  Args a(env, info);
  uint64_t e;
  if (a.argc < 1 || !get_u64(env, a.argv[0], &e)) { napi_throw_type_error(env, nullptr, "eventDestroy(event)"); return nullptr; }
  JH_OK(jh_event_destroy((jh_event)(uintptr_t)e));
  return nullptr;
}

napi_value GraphBegin(napi_env env, napi_callback_info) {  // launches queued until graphEnd() are recorded, not run
  JH_OK(jh_graph_begin());
  return nullptr;
}

napi_value GraphEnd(napi_env env, napi_callback_info) {  // -> BigInt graph handle
  jh_graph g = nullptr;
  JH_OK(jh_graph_end(&g));
  return make_u64(env, (uint64_t)(uintptr_t)g);
}

napi_value GraphLaunch(napi_env env, napi_callback_info info) {
  Args a(env, info);
  uint64_t g;
  if (a.argc < 1 || !get_u64(env, a.argv[0], &g)) { napi_throw_type_error(env, nullptr, "graphLaunch(graph)"); return nullptr; }
  JH_OK(jh_graph_launch((jh_graph)(uintptr_t)g));
  return nullptr;
}

napi_value GraphDestroy(napi_env env, napi_callback_info info) {
  Args a(env, info);
  uint64_t g;
  if (a.argc < 1 || !get_u64(env, a.argv[0], &g)) { napi_throw_type_error(env, nullptr, "graphDestroy(graph)"); return nullptr; }
  JH_OK(jh_graph_destroy((jh_graph)(uintptr_t)g));
  return nullptr;
}

napi_value AbiVersion(napi_env env, napi_callback_info) {
  napi_value out;
  napi_create_int32(env, jh_abi_version(), &out);
  return out;
}

}  // namespace

NAPI_MODULE_INIT() {
  const struct { const char* name; napi_callback fn; } table[] = {
      {"init", Init}, {"shutdown", Shutdown}, {"deviceInfo", DeviceInfo}, {"malloc", Malloc}, {"free", Free},
      {"h2d", H2D}, {"d2h", D2H}, {"compile", Compile}, {"moduleLoad", ModuleLoad}, {"moduleUnload", ModuleUnload},
      {"moduleFunction", ModuleFunction}, {"launch", Launch}, {"sync", Sync}, {"eventCreate", EventCreate},
      {"eventRecord", EventRecord}, {"eventQuery", EventQuery}, {"eventElapsedMs", EventElapsed},
      {"eventDestroy", EventDestroy}, {"graphBegin", GraphBegin}, {"graphEnd", GraphEnd}, {"graphLaunch", GraphLaunch},
      {"graphDestroy", GraphDestroy}, {"abiVersion", AbiVersion}, {"d2hAsync", D2HAsync}, {"compilerVersion", CompilerVersion},
      {"d2d", D2D},
  };
  for (const auto& e : table) {
    napi_value fn;
    if (napi_create_function(env, e.name, NAPI_AUTO_LENGTH, e.fn, nullptr, &fn) != napi_ok) return nullptr;
    if (napi_set_named_property(env, exports, e.name, fn) != napi_ok) return nullptr;
  }
  return exports;
}

/*
 * jaxhip.h -- C ABI of the MI355X runtime under the jax-js `hip` backend.
 *
 * This is the only native surface the host-side `HipBackend` (the object that implements the
 * reference's `Backend` interface, src/backend.ts:158-211) talks to.  The host side owns slots,
 * reference counts, the kernel cache and code generation; this library owns the device: memory,
 * one in-order stream, run-time compilation (hiprtc) and kernel launches.  Plain pointers and
 * sizes only, so that it can be bound from an N-API addon, ctypes, cgo or JNI alike.
 *
 * Conventions
 *   - Every function returns 0 on success and a non-zero status on failure; `jh_last_error()`
 *     returns a message for the most recent failure on the calling thread.  The host layer turns
 *     a failure into the exception the reference's interface prescribes (src/backend.ts:222-240).
 *   - All work is issued on one stream in call order, which is what gives `Backend.dispatch`
 *     its "operations run in dispatch order" guarantee (src/backend.ts:203-210).
 *   - One caller thread is assumed, as in the reference (a single JS thread).
 */
#ifndef JAXHIP_H
#define JAXHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *jh_devptr;   /* device address */
typedef void *jh_module;   /* loaded code object */
typedef void *jh_function; /* kernel entry point inside a module */
typedef void *jh_event;    /* timing / completion marker on the stream */

typedef struct jh_device_info {
  char name[128];      /* marketing name */
  char arch[64];       /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
  int32_t compute_units;
  int32_t wavefront_size;
  int32_t max_threads_per_block;
  int32_t lds_bytes_per_block;
  int64_t total_mem_bytes;
  int32_t clock_khz;
  int32_t l2_bytes;
} jh_device_info;

/*
 * Bring the device up: select it, create the stream.  Replaces the per-backend construction in
 * `createBackend(device)` (src/backend.ts:72-142; the WebGPU arm requests an adapter and device
 * there).  Calling it again for the same device is a no-op.
 */
int jh_init(int device);

/* Tear down the stream and forget cached state.  (No counterpart: JS backends are GC'd.) */
int jh_shutdown(void);

/* Device properties, for the tuner's tile/wave choices (the WebGPU backend reads
 * `device.limits` for the same purpose, src/backend/webgpu.ts:331-340). */
int jh_get_device_info(jh_device_info *out);

/*
 * Raw device memory.  Backs `Backend.malloc` / the free at refcount zero in `Backend.decRef`
 * (src/backend.ts:170-179; `device.createBuffer` / `buffer.destroy` in src/backend/webgpu.ts:224-247).
 * `bytes == 0` yields a NULL pointer and success.
 */
int jh_malloc(size_t bytes, jh_devptr *out);
int jh_free(jh_devptr ptr);

/*
 * Host -> device upload of `initialData` in `Backend.malloc` (src/backend.ts:170;
 * `queue.writeBuffer` in the WebGPU backend).  Ordered with kernels on the stream; the host
 * buffer may be reused as soon as the call returns.
 */
int jh_memcpy_h2d(jh_devptr dst, const void *src, size_t bytes);

/*
 * Device -> host read of `bytes` starting `offset` bytes into `src`.  Backs `Backend.readSync`
 * (src/backend.ts:189): returns after every previously issued kernel has finished.  Reads of
 * 1 MiB and more are pipelined through two pinned 8 MiB buffers that the library allocates at the
 * first such read and keeps until `jh_shutdown`.  Those two buffers are shared by every call: the
 * function is not reentrant, call it from one thread at a time (as every other entry point).
 */
int jh_memcpy_d2h(void *dst, jh_devptr src, size_t offset, size_t bytes);

/*
 * Asynchronous flavour backing `Backend.read` (src/backend.ts:182-186; staging-buffer map in
 * src/backend/webgpu/reader.ts): the copy is queued and `*done` is an event to poll with
 * `jh_event_query` or wait on with `jh_event_sync`.  `dst` must stay valid until then and should
 * come from `jh_host_alloc` for a truly asynchronous copy.
 */
int jh_memcpy_d2h_async(void *dst, jh_devptr src, size_t offset, size_t bytes, jh_event *done);

/* Device -> device copy on the stream (used when a routine result is moved into an output slot). */
int jh_memcpy_d2d(jh_devptr dst, jh_devptr src, size_t bytes);

/* Pinned host memory for asynchronous reads.  `jh_host_free` also works after `jh_shutdown` (a garbage collector
 * may return a staging buffer late). */
int jh_host_alloc(size_t bytes, void **out);
int jh_host_free(void *ptr);

/*
 * Compile HIP source text to a gfx950 code object with hiprtc.  Replaces shader compilation in
 * `prepareKernel` (src/backend.ts:192-195; `createComputePipelineAsync` in
 * src/backend/webgpu.ts:705-744, `new WebAssembly.Module` in src/backend/wasm.ts:125-147).
 * Needs no GPU, so it can also run ahead of time.  On success `*code`/`*code_size` hold a
 * malloc'd code object to release with `jh_code_free`; on failure `log` (if non-NULL) receives
 * the compiler output, truncated to `log_size`.  A source may ask for options of its own in leading lines of the form
 * `// hiprtc-option: <option>`: they are added to `options` when they are on the library's fixed list
 * (`-fno-slp-vectorize`, which the generator puts on float16 kernels) and make the call fail when they are not.
 */
int jh_compile(const char *source, const char *name, const char *const *options, int num_options,
               void **code, size_t *code_size, char *log, size_t log_size);
void jh_code_free(void *code);

/* Version of the run-time compiler behind `jh_compile` (hiprtcVersion).  The host side mixes it into the key of its
 * on-disk code-object cache, so that a toolchain change never reuses stale code objects (the WebGPU backend's
 * pipeline cache is keyed by shader text alone because the browser owns the compiler, src/backend/webgpu.ts:705-744). */
int jh_compiler_version(int *major, int *minor);

/* Load a code object on the device and look up a kernel in it. */
int jh_module_load(const void *code, size_t code_size, jh_module *out);
int jh_module_unload(jh_module module);
int jh_module_function(jh_module module, const char *kernel_name, jh_function *out);

/*
 * Queue one kernel launch.  Backs `Backend.dispatch` (src/backend.ts:203-210;
 * `dispatchWorkgroups` in src/backend/webgpu.ts:532-618).  `args[i]` points at the i-th kernel
 * parameter (device pointers and scalars), exactly as `hipModuleLaunchKernel` takes them.
 * Never blocks on the device.
 */
int jh_launch(jh_function fn, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z, uint32_t block_x,
              uint32_t block_y, uint32_t block_z, uint32_t shared_bytes, void **args);

/*
 * `jh_launch` for callers that cannot allocate (a launch recorded under graph capture, a serving loop, a harness that
 * forbids hipMalloc).  No counterpart in the reference.  Kernels whose reduce axis is cut over several workgroups
 * (two-stage reductions, split-k GEMMs) write partial accumulators to a scratch buffer that the host side normally
 * allocates per executable; here the kernel argument number `scratch_arg` is instead pointed at a buffer that lives
 * inside the library (a file-scope device array of `jh_static_scratch_bytes` = 32 MiB per GPU, held until the process
 * ends): the 8-byte cell `args[scratch_arg]` points at is overwritten with its device address, then the launch is
 * queued exactly like `jh_launch`.  `scratch_bytes` is what the kernel will address; more than the buffer holds is an
 * error and nothing is launched.  Calls no hipMalloc/hipFree.  Every call on a GPU shares that GPU's buffer, which
 * keeps the previous call's contents (these kernels write every partial before reading it, so nothing needs clearing);
 * launches that use it must not overlap -- on this library's single in-order stream they never do.
 */
int jh_launch_static_scratch(jh_function fn, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z, uint32_t block_x,
                             uint32_t block_y, uint32_t block_z, uint32_t shared_bytes, void **args,
                             uint32_t scratch_arg, size_t scratch_bytes);
int jh_static_scratch_bytes(size_t *bytes);

/* Same launch repeated `count` times back to back (benchmark loops without per-call host overhead). */
int jh_launch_repeat(jh_function fn, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z, uint32_t block_x,
                     uint32_t block_y, uint32_t block_z, uint32_t shared_bytes, void **args, int count);

/*
 * Record a sequence of launches once and replay it with one call.  Everything queued with `jh_launch` between
 * `jh_graph_begin` and `jh_graph_end` is captured into a HIP graph instead of running; `jh_graph_launch`
 * then replays the whole sequence in order on the stream.  This is how a compiled jit program
 * (`JitProgram.execute`, src/frontend/jit.ts:111-162: a fixed list of kernel dispatches over fixed
 * buffers) is issued without per-kernel host work.  No allocation, copy or synchronisation call may be made
 * while a capture is open; buffers the launches name must stay allocated for the graph's lifetime.
 */
typedef void *jh_graph;
int jh_graph_begin(void);
int jh_graph_end(jh_graph *out);
int jh_graph_launch(jh_graph graph);
int jh_graph_destroy(jh_graph graph);

/* Wait for everything queued so far (the completion fence `read(slot, 0, 0)` stands for in
 * src/frontend/array.ts:827). */
int jh_sync(void);

/*
 * Events on the stream: the profiler hook's timestamps (the WebGPU backend brackets each pass with
 * `timestamp-query` pairs, src/backend/webgpu/tracing.ts:11-60) and the completion handles of
 * asynchronous reads.
 */
int jh_event_create(jh_event *out);
int jh_event_record(jh_event ev);
int jh_event_query(jh_event ev, int *done);           /* non-blocking */
int jh_event_sync(jh_event ev);                       /* blocking */
int jh_event_elapsed_ms(jh_event start, jh_event stop, float *ms);
int jh_event_destroy(jh_event ev);

/* Message for the most recent failure on this thread ("" if none). */
const char *jh_last_error(void);

/* ABI version of this header: bumped whenever a signature changes. */
int jh_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif /* JAXHIP_H */

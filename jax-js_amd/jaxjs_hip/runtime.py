"""ctypes binding of the C-ABI runtime (`include/jaxhip.h`, built as `csrc/libjaxhip.so`).

The only module that touches native code.  Fails loudly when the library is missing or the device
cannot be initialised: there is no CPU fallback behind the `hip` backend.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import threading

import numpy as np
from typing import List, Optional, Sequence, Tuple

from .codegen import SOURCE_OPTION, SOURCE_OPTIONS_ALLOWED
from .errors import HipRuntimeError

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG, "csrc", "libjaxhip.so")
CACHE_DIR = os.environ.get("JAXHIP_KERNEL_CACHE", os.path.join(_PKG, "kcache"))

# Options every kernel is compiled with.  -ffp-contract=off keeps f32 arithmetic bit-faithful to
# the expression (fused multiply-adds are written explicitly where wanted); packed-fp32 VALU ops
# are disabled on this hardware pool.
COMPILE_OPTIONS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 128),
        ("arch", ctypes.c_char * 64),
        ("compute_units", ctypes.c_int32),
        ("wavefront_size", ctypes.c_int32),
        ("max_threads_per_block", ctypes.c_int32),
        ("lds_bytes_per_block", ctypes.c_int32),
        ("total_mem_bytes", ctypes.c_int64),
        ("clock_khz", ctypes.c_int32),
        ("l2_bytes", ctypes.c_int32),
    ]


_SIGNATURES = {
    "jh_abi_version": (ctypes.c_int, []),
    "jh_last_error": (ctypes.c_char_p, []),
    "jh_init": (ctypes.c_int, [ctypes.c_int]),
    "jh_shutdown": (ctypes.c_int, []),
    "jh_get_device_info": (ctypes.c_int, [ctypes.POINTER(DeviceInfo)]),
    "jh_malloc": (ctypes.c_int, [ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]),
    "jh_free": (ctypes.c_int, [ctypes.c_void_p]),
    "jh_memcpy_h2d": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
    "jh_memcpy_d2h": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]),
    "jh_memcpy_d2h_async": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t,
                                           ctypes.POINTER(ctypes.c_void_p)]),
    "jh_memcpy_d2d": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
    "jh_host_alloc": (ctypes.c_int, [ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]),
    "jh_host_free": (ctypes.c_int, [ctypes.c_void_p]),
    "jh_compile": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_char_p), ctypes.c_int,
                                  ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_size_t),
                                  ctypes.c_char_p, ctypes.c_size_t]),
    "jh_code_free": (None, [ctypes.c_void_p]),
    "jh_compiler_version": (ctypes.c_int, [ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]),
    "jh_module_load": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]),
    "jh_module_unload": (ctypes.c_int, [ctypes.c_void_p]),
    "jh_module_function": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]),
    "jh_launch": (ctypes.c_int, [ctypes.c_void_p] + [ctypes.c_uint32] * 7 + [ctypes.POINTER(ctypes.c_void_p)]),
    "jh_launch_static_scratch": (ctypes.c_int, [ctypes.c_void_p] + [ctypes.c_uint32] * 7 +
                                 [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint32, ctypes.c_size_t]),
    "jh_static_scratch_bytes": (ctypes.c_int, [ctypes.POINTER(ctypes.c_size_t)]),
    "jh_launch_repeat": (ctypes.c_int, [ctypes.c_void_p] + [ctypes.c_uint32] * 7 +
                         [ctypes.POINTER(ctypes.c_void_p), ctypes.c_int]),
    "jh_sync": (ctypes.c_int, []),
    "jh_graph_begin": (ctypes.c_int, []),
    "jh_graph_end": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p)]),
    "jh_graph_launch": (ctypes.c_int, [ctypes.c_void_p]),
    "jh_graph_destroy": (ctypes.c_int, [ctypes.c_void_p]),
    "jh_event_create": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p)]),
    "jh_event_record": (ctypes.c_int, [ctypes.c_void_p]),
    "jh_event_query": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]),
    "jh_event_sync": (ctypes.c_int, [ctypes.c_void_p]),
    "jh_event_elapsed_ms": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_float)]),
    "jh_event_destroy": (ctypes.c_int, [ctypes.c_void_p]),
}

EXPORTED_SYMBOLS = sorted(_SIGNATURES)

_lib: Optional[ctypes.CDLL] = None


def load_library() -> ctypes.CDLL:
    """dlopen libjaxhip.so and type its entry points (no device work)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipRuntimeError(
            f"native runtime not built: {LIB_PATH} is missing (run `python -c 'import __graft_entry__ as g; g.build()'`)"
        )
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as e:
        raise HipRuntimeError(f"cannot load {LIB_PATH}: {e}") from e
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load_library().jh_last_error().decode(errors="replace")
        raise HipRuntimeError(f"{what} failed (status {rc}): {msg}")


_toolchain: Optional[str] = None


def toolchain_tag() -> str:
    """What a cached code object depends on besides its source and options: the run-time compiler's version and this
    library's ABI version.  (The target architecture is one of the options.)"""
    global _toolchain
    if _toolchain is None:
        lib = load_library()
        major, minor = ctypes.c_int(), ctypes.c_int()
        check(lib.jh_compiler_version(ctypes.byref(major), ctypes.byref(minor)), "jh_compiler_version")
        _toolchain = f"hiprtc-{major.value}.{minor.value}/abi-{lib.jh_abi_version()}"
    return _toolchain


DISK_CACHE = os.environ.get("JAXHIP_NO_DISK_CACHE") != "1"  # False: every prepare goes through hiprtc


def compile_source(source: str, name: str = "kernel.hip", options: Optional[Sequence[str]] = None,
                   use_cache: Optional[bool] = None) -> bytes:
    """HIP source -> gfx950 code object through hiprtc, with an on-disk cache keyed by compiler version, options
    and source text."""
    lib = load_library()
    if use_cache is None:
        use_cache = DISK_CACHE
    opts = list(options if options is not None else COMPILE_OPTIONS)
    for line in source.split("\n", 4)[:4]:  # options the generator asks for in the source's opening lines
        if line.startswith(SOURCE_OPTION):
            opt = line[len(SOURCE_OPTION):].strip()
            if opt not in SOURCE_OPTIONS_ALLOWED:
                raise HipRuntimeError(f"{name}: the source asks for a compiler option that is not on the list: {opt!r}")
            if opt not in opts:
                opts.append(opt)
    key = hashlib.sha256((toolchain_tag() + "\0" + "\0".join(opts) + "\0" + source).encode()).hexdigest()[:32]
    path = os.path.join(CACHE_DIR, key + ".hsaco")
    if use_cache and os.path.exists(path):
        with open(path, "rb") as f:
            return f.read()
    arr = (ctypes.c_char_p * len(opts))(*[o.encode() for o in opts])
    code = ctypes.c_void_p()
    size = ctypes.c_size_t()
    log = ctypes.create_string_buffer(1 << 16)
    rc = lib.jh_compile(source.encode(), name.encode(), arr, len(opts), ctypes.byref(code), ctypes.byref(size),
                        log, len(log))
    if rc != 0:
        text = log.value.decode(errors="replace") or lib.jh_last_error().decode(errors="replace")
        raise HipRuntimeError(f"hiprtc failed for {name} (status {rc}):\n{text}")
    try:
        blob = ctypes.string_at(code, size.value)
    finally:
        lib.jh_code_free(code)
    if use_cache:
        try:
            os.makedirs(CACHE_DIR, exist_ok=True)
            tmp = path + f".tmp{os.getpid()}.{threading.get_ident()}"  # compilations run on several threads
            with open(tmp, "wb") as f:
                f.write(blob)
            os.replace(tmp, path)
        except OSError:
            pass
    return blob


class Device:
    """The initialised device: memory, modules, launches, events.  One per process."""

    _instance: Optional["Device"] = None

    def __init__(self, index: int = 0):
        self.lib = load_library()
        check(self.lib.jh_init(index), "jh_init")
        info = DeviceInfo()
        check(self.lib.jh_get_device_info(ctypes.byref(info)), "jh_get_device_info")
        self.info = info
        self.arch = info.arch.decode()
        self.name = info.name.decode()

    @classmethod
    def get(cls, index: int = 0) -> "Device":
        if cls._instance is None:
            cls._instance = Device(index)
        return cls._instance

    # -- memory ---------------------------------------------------------------------------------
    def malloc(self, nbytes: int) -> int:
        p = ctypes.c_void_p()
        check(self.lib.jh_malloc(nbytes, ctypes.byref(p)), f"jh_malloc({nbytes})")
        return p.value or 0

    def free(self, ptr: int) -> None:
        if ptr:
            check(self.lib.jh_free(ctypes.c_void_p(ptr)), "jh_free")

    def h2d(self, dst: int, data) -> None:
        mv = memoryview(data).cast("B")
        if len(mv) == 0:
            return
        src = np.frombuffer(mv, dtype=np.uint8)  # the buffer's own address, read-only or not: no host-side copy
        check(self.lib.jh_memcpy_h2d(ctypes.c_void_p(dst), ctypes.c_void_p(src.ctypes.data), len(mv)), "jh_memcpy_h2d")

    def d2h(self, src: int, offset: int, nbytes: int) -> bytearray:
        out = bytearray(nbytes)
        if nbytes:
            buf = (ctypes.c_char * nbytes).from_buffer(out)
            check(self.lib.jh_memcpy_d2h(ctypes.cast(buf, ctypes.c_void_p), ctypes.c_void_p(src), offset, nbytes),
                  "jh_memcpy_d2h")
        else:
            check(self.lib.jh_memcpy_d2h(None, None, 0, 0), "jh_memcpy_d2h")
        return out

    def host_alloc(self, nbytes: int) -> int:
        """Pinned host memory (the destination of asynchronous reads)."""
        p = ctypes.c_void_p()
        check(self.lib.jh_host_alloc(nbytes, ctypes.byref(p)), f"jh_host_alloc({nbytes})")
        return p.value or 0

    def host_free(self, ptr: int) -> None:
        if ptr:
            check(self.lib.jh_host_free(ctypes.c_void_p(ptr)), "jh_host_free")

    def d2h_async(self, host_ptr: int, src: int, offset: int, nbytes: int) -> int:
        """Queue a device -> pinned-host copy behind everything issued so far; returns the completion event."""
        ev = ctypes.c_void_p()
        check(self.lib.jh_memcpy_d2h_async(ctypes.c_void_p(host_ptr), ctypes.c_void_p(src), offset, nbytes, ctypes.byref(ev)),
              "jh_memcpy_d2h_async")
        return ev.value

    def event_done(self, ev: int) -> bool:
        done = ctypes.c_int()
        check(self.lib.jh_event_query(ctypes.c_void_p(ev), ctypes.byref(done)), "jh_event_query")
        return bool(done.value)

    def d2d(self, dst: int, src: int, nbytes: int) -> None:
        check(self.lib.jh_memcpy_d2d(ctypes.c_void_p(dst), ctypes.c_void_p(src), nbytes), "jh_memcpy_d2d")

    # -- code -----------------------------------------------------------------------------------
    def load_module(self, code: bytes) -> int:
        m = ctypes.c_void_p()
        check(self.lib.jh_module_load(code, len(code), ctypes.byref(m)), "jh_module_load")
        return m.value

    def unload_module(self, module: int) -> None:
        check(self.lib.jh_module_unload(ctypes.c_void_p(module)), "jh_module_unload")

    def function(self, module: int, name: str) -> int:
        f = ctypes.c_void_p()
        check(self.lib.jh_module_function(ctypes.c_void_p(module), name.encode(), ctypes.byref(f)),
              f"jh_module_function({name})")
        return f.value

    def launch(self, fn: int, grid, block, shared: int, argv, repeat: int = 1) -> None:
        if repeat == 1:
            rc = self.lib.jh_launch(ctypes.c_void_p(fn), grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                    shared, argv)
        else:
            rc = self.lib.jh_launch_repeat(ctypes.c_void_p(fn), grid[0], grid[1], grid[2], block[0], block[1],
                                           block[2], shared, argv, repeat)
        check(rc, "jh_launch")

    def sync(self) -> None:
        check(self.lib.jh_sync(), "jh_sync")

    # -- graphs ---------------------------------------------------------------------------------
    def graph_begin(self) -> None:
        check(self.lib.jh_graph_begin(), "jh_graph_begin")

    def graph_end(self) -> int:
        g = ctypes.c_void_p()
        check(self.lib.jh_graph_end(ctypes.byref(g)), "jh_graph_end")
        return g.value

    def graph_launch(self, graph: int) -> None:
        check(self.lib.jh_graph_launch(ctypes.c_void_p(graph)), "jh_graph_launch")

    def graph_destroy(self, graph: int) -> None:
        check(self.lib.jh_graph_destroy(ctypes.c_void_p(graph)), "jh_graph_destroy")

    # -- events ---------------------------------------------------------------------------------
    def event(self) -> int:
        e = ctypes.c_void_p()
        check(self.lib.jh_event_create(ctypes.byref(e)), "jh_event_create")
        return e.value

    def record(self, ev: int) -> None:
        check(self.lib.jh_event_record(ctypes.c_void_p(ev)), "jh_event_record")

    def elapsed_ms(self, start: int, stop: int) -> float:
        check(self.lib.jh_event_sync(ctypes.c_void_p(stop)), "jh_event_sync")
        ms = ctypes.c_float()
        check(self.lib.jh_event_elapsed_ms(ctypes.c_void_p(start), ctypes.c_void_p(stop), ctypes.byref(ms)),
              "jh_event_elapsed_ms")
        return ms.value

    def destroy_event(self, ev: int) -> None:
        check(self.lib.jh_event_destroy(ctypes.c_void_p(ev)), "jh_event_destroy")


def pack_args(values: Sequence[int]):
    """kernelParams array for 8-byte arguments (device pointers, integers): returns (argv, keepalive).
    One array holds the values and one the addresses of its cells; a plan of hundreds of small launches
    (LU by columns, staged FFT) is bound by this host work, so no per-argument ctypes object is made."""
    n = len(values)
    cells = (ctypes.c_uint64 * n)(*values)
    base = ctypes.addressof(cells)
    argv = (ctypes.c_void_p * n)(*[base + 8 * i for i in range(n)])
    return argv, cells

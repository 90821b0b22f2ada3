"""`jh_launch_static_scratch`: the launch entry point that allocates nothing.  Kernels that keep partial results in a
scratch buffer (a two-stage reduction, a split-k GEMM) run through it on the library's static scratch array and must
give the bytes the ordinary `jh_launch` path gives on the executable's own hipMalloc'ed scratch: two calls in a row,
the second on a smaller input (the static buffer still holds the first call's partials)."""
import ctypes

import numpy as np
import pytest

from gpu_util import WARM_ONLY, backend
from jaxjs_hip import AluOp, DType, ShapeTracker, numpyDtype
from jaxjs_hip.lowering import matmulKernel, reduceKernel

pytestmark = pytest.mark.gpu
F32 = DType.Float32


def _both_ways(be, kernel, host, **tune):
    exe = be.prepareKernelSync(kernel, **tune)
    ks = exe.data.ks
    assert len(ks.scratch_bytes) == 1 and any(kind == "scratch" for st in ks.steps for kind, _ in st.args), ks.klass
    slots = [be.malloc(np.ascontiguousarray(x).nbytes, np.ascontiguousarray(x).tobytes()) for x in host]
    o1, o2 = be.malloc(kernel.bytes), be.malloc(kernel.bytes)
    try:
        be.dispatch(exe, slots, [o1])
        be.dispatchStaticScratch(exe, slots, [o2])
        a = np.frombuffer(be.readSync(o1), dtype=numpyDtype(kernel.dtype)).copy()
        b = np.frombuffer(be.readSync(o2), dtype=numpyDtype(kernel.dtype)).copy()
        be.dispatch(exe, slots, [o1])  # the ordinary path still works on its own scratch afterwards
        a2 = np.frombuffer(be.readSync(o1), dtype=numpyDtype(kernel.dtype)).copy()
    finally:
        for s in slots + [o1, o2]:
            be.decRef(s)
    np.testing.assert_array_equal(a, a2)
    return a, b, ks


def test_static_scratch_matches_allocated_scratch_twice_in_a_row():
    if WARM_ONLY:
        pytest.skip("warm-up run")
    be = backend()
    rng = np.random.default_rng(21)
    for n in (1 << 24, 1 << 21):  # flat sums cut over many workgroups; the second, smaller call reuses the buffer
        x = rng.normal(0, 1, n).astype(np.float32)
        k = reduceKernel([1, n], [(F32, ShapeTracker.fromShape([1, n]))], lambda v: v, AluOp.Add)
        a, b, ks = _both_ways(be, k, [x])
        assert ks.klass == "reduce_row+fold"
        np.testing.assert_array_equal(a, b)  # same kernels, same fold order: the same bits
        assert abs(float(a[0]) - float(np.sum(x.astype(np.float64)))) <= 2 * n * np.finfo(np.float32).eps * float(np.abs(x).sum())
    for (M, N, K) in ((256, 512, 2048), (128, 256, 512)):  # split-k GEMMs: f32 partials [slice][M*N]
        A = rng.uniform(-1, 1, (M, K)).astype(np.float16)
        B = rng.uniform(-1, 1, (K, N)).astype(np.float16)
        k = matmulKernel(M, N, K, DType.Float16)
        # the fold of the slices by a second kernel: the in-launch fold keeps counters in a second scratch buffer
        a, b, ks = _both_ways(be, k, [A, B], gemm_tile=(("FUSEK", 0), ("SPLITK", 4)))
        assert ks.klass == "gemm+fold" and ks.info["splitk"] == 4
        np.testing.assert_array_equal(a, b)
        ref = A.astype(np.float64) @ B.astype(np.float64)
        np.testing.assert_allclose(a.reshape(M, N).astype(np.float64), ref, rtol=2e-3, atol=2e-2)


def test_static_scratch_rejects_oversized_requests_without_launching():
    if WARM_ONLY:
        pytest.skip("warm-up run")
    be = backend()
    lib = be.dev.lib
    cap = ctypes.c_size_t()
    assert lib.jh_static_scratch_bytes(ctypes.byref(cap)) == 0 and cap.value == 32 << 20
    n = 1 << 16
    k = reduceKernel([1, n], [(F32, ShapeTracker.fromShape([1, n]))], lambda v: v, AluOp.Add)
    exe = be.prepareKernelSync(k)
    head, (cells, argv, patch) = exe.data.launch_head[0], exe.data.bound[0]
    before = cells[len(cells) - 1]
    rc = lib.jh_launch_static_scratch(*head, argv, len(cells) - 1, cap.value + 1)
    assert rc != 0 and b"static scratch" in lib.jh_last_error() and cells[len(cells) - 1] == before
    # a GEMM whose partials exceed the buffer is refused by the host layer through the same status
    M, N, K = 4096, 4096, 512
    kk = matmulKernel(M, N, K, DType.Float16)
    big = be.prepareKernelSync(kk, gemm_tile=(("SPLITK", 2),))
    assert big.data.ks.scratch_bytes[0] > cap.value
    a, b, o = be.malloc(M * K * 2), be.malloc(K * N * 2), be.malloc(kk.bytes)
    try:
        with pytest.raises(Exception, match="static scratch"):
            be.dispatchStaticScratch(big, [a, b], [o])
    finally:
        for s in (a, b, o):
            be.decRef(s)


def test_static_scratch_refuses_executables_with_state_in_a_second_scratch_buffer():
    """A k split folded inside the launch keeps per-tile arrival counters in a second scratch buffer that must start at
    zero: one shared static buffer cannot serve it, and the host layer says so before anything is launched."""
    if WARM_ONLY:
        pytest.skip("warm-up run")
    be = backend()
    k = matmulKernel(1024, 1024, 1024, F32)
    exe = be.prepareKernelSync(k)
    assert exe.data.ks.info.get("fused_fold") and len(exe.data.ks.scratch_bytes) == 2
    a, b, o = be.malloc(4 << 20), be.malloc(4 << 20), be.malloc(k.bytes)
    try:
        with pytest.raises(ValueError, match="several scratch buffers"):
            be.dispatchStaticScratch(exe, [a, b], [o])
    finally:
        for s in (a, b, o):
            be.decRef(s)

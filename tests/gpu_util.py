"""Shared helpers for the GPU parity tests: run a Kernel through the C-ABI path and through the CPU checker."""
import os

import numpy as np
import pytest

from jaxjs_hip import numpyDtype
from oracle import oracle

WARM_ONLY = os.environ.get("JAXHIP_WARM") == "1"  # compile every kernel into the on-disk cache, run nothing

_backends = {}
NUMERICS = "wasm"  # the mode `backend()` hands out; the `numerics_mode` fixture of a test module switches it


def set_numerics(mode):
    global NUMERICS
    NUMERICS = mode


def backend():
    """The backend the parity tests run on.  By default Wasm-faithful numerics, so that f32 maps can be held to 2 ulp of
    the checker; test modules that carry the `numerics_mode` fixture run a second time on the backend's own default,
    "fast" (exp and reciprocal on hardware instructions, within rel 1e-5 of the checker)."""
    if "wasm" not in _backends:
        from jaxjs_hip import getBackend, init

        init("hip", numerics="wasm")
        _backends["wasm"] = getBackend("hip")
    if NUMERICS not in _backends:
        from jaxjs_hip.backend import HipBackend

        _backends[NUMERICS] = HipBackend(numerics=NUMERICS)
        assert _backends[NUMERICS].numerics == NUMERICS
    return _backends[NUMERICS]


def fast_backend():
    """A second backend object on the same device with the default ("fast") numerics."""
    from jaxjs_hip.backend import HipBackend

    backend()
    if "fast" not in _backends:
        _backends["fast"] = HipBackend()
        assert _backends["fast"].numerics == "fast"
    return _backends["fast"]


def device_run(kernel, inputs, **tune_opts):
    """Upload inputs, dispatch the kernel once, read the typed result back."""
    if WARM_ONLY:
        from jaxjs_hip.kernelgen import generate
        from jaxjs_hip.runtime import compile_source

        for src in generate(kernel, NUMERICS, **tune_opts).sources:
            compile_source(src)
        pytest.skip("warm-up run: compiled only")
    be = backend()
    exe = be.prepareKernelSync(kernel, **tune_opts)
    slots = []
    for x in inputs:
        a = np.ascontiguousarray(x)
        slots.append(be.malloc(a.nbytes, a.tobytes()))
    out = be.malloc(kernel.bytes)
    try:
        be.dispatch(exe, slots, [out])
        raw = be.readSync(out)
    finally:
        for s in slots + [out]:
            be.decRef(s)
    return np.frombuffer(raw, dtype=numpyDtype(kernel.dtype)).copy(), exe.data.ks


def ulp_diff_f32(a, b):
    """Distance in units of f32 representation between two float32 arrays (NaNs must coincide)."""
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    nan = np.isnan(a) | np.isnan(b)
    assert np.array_equal(np.isnan(a), np.isnan(b)), "NaN positions differ"
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia)
    ib = np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    d = np.abs(ia - ib)
    d[nan] = 0
    return d


def assert_parity(kernel, inputs, *, exact=False, rtol=1e-5, atol=1e-7, mode=oracle.MODE_WASM, max_ulp=None, **tune_opts):
    got, ks = device_run(kernel, inputs, **tune_opts)
    want = oracle.run_kernel(kernel, inputs, mode)
    assert got.dtype == want.dtype and got.shape == want.shape
    if exact or got.dtype.kind in "iu":
        np.testing.assert_array_equal(got, want, err_msg=f"class {ks.klass} {ks.info}")
    else:
        np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=rtol, atol=atol, equal_nan=True,
                                   err_msg=f"class {ks.klass} {ks.info}")
        if max_ulp is not None and got.dtype == np.float32:
            assert ulp_diff_f32(got, want).max() <= max_ulp
    return got, want, ks

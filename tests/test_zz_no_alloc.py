"""cthip_matmul_noalloc, the entry point for callers that cannot allocate device memory: through the C ABI it must
give what cthip_matmul gives (same kernels, same split of the reduction, partial tiles in the library's static
scratch instead of an allocator block) -- bit for bit, and within rtol 1e-3 / atol 1e-4 of an fp64 product -- on
two calls in a row, the second smaller than the first (the scratch keeps the first call's partial tiles), while
the allocator sees no traffic; a shape whose partial tiles exceed the scratch is refused."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-3, 1e-4


def _run(lib, check, fn, A, B, act, precision):
    from caten_amd import ops
    M, K = A.shape
    N = B.shape[1]
    dA, dB = ops.DeviceArray.from_numpy(A), ops.DeviceArray.from_numpy(B)
    dC = ops.DeviceArray((M, N), np.float32)
    live0, cached0, drv0 = C.c_size_t(), C.c_size_t(), C.c_size_t()
    check(lib.cthip_cache_stats(C.byref(live0), C.byref(cached0), C.byref(drv0)))
    check(fn(dC.ptr, dA.ptr, dB.ptr, M, N, K, act, precision))
    live1, cached1, drv1 = C.c_size_t(), C.c_size_t(), C.c_size_t()
    check(lib.cthip_cache_stats(C.byref(live1), C.byref(cached1), C.byref(drv1)))
    out = dC.numpy()
    return out, (live1.value - live0.value, cached1.value - cached0.value, drv1.value - drv0.value)


@pytest.mark.parametrize("precision", [0, 3])
def test_noalloc_matmul_equals_matmul_twice_in_a_row(precision):
    from caten_amd import _lib
    lib = _lib.init(0)
    rng = np.random.default_rng(7)
    # both shapes split their reduction (few tiles, long K), so both use the scratch; the second is smaller
    for (M, N, K) in [(256, 256, 2048), (130, 190, 1024)]:
        print(f"case: matmul_noalloc {M}x{N}x{K} precision {precision}", flush=True)
        A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
        want, _ = _run(lib, _lib.check, lib.cthip_matmul, A, B, 1, precision)
        got, delta = _run(lib, _lib.check, lib.cthip_matmul_noalloc, A, B, 1, precision)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        assert delta == (0, 0, 0), f"the allocator moved during the call: {delta}"
        ref = np.maximum(A.astype(np.float64) @ B.astype(np.float64), 0.0)
        bad = np.abs(got - ref) > ATOL + RTOL * np.abs(ref)
        assert not bad.any()


def test_noalloc_matmul_refuses_what_the_scratch_cannot_hold():
    from caten_amd import _lib, HipError, ops
    lib = _lib.init(0)
    M = N = 512
    K = 4096  # 64 tiles: the reduction is split eight ways, 8 x 512 x 512 x 4 bytes of partial tiles
    dA, dB = ops.DeviceArray((M, K), np.float32), ops.DeviceArray((K, N), np.float32)
    dC = ops.DeviceArray((M, N), np.float32)
    with pytest.raises(HipError, match="static scratch"):
        _lib.check(lib.cthip_matmul_noalloc(dC.ptr, dA.ptr, dB.ptr, M, N, K, 0, 0))
    _lib.check(lib.cthip_matmul(dC.ptr, dA.ptr, dB.ptr, M, N, K, 0, 0))  # the allocating entry point takes it
    _lib.check(lib.cthip_sync())

"""The sort entry point that allocates nothing (pccnn_sort_keys_static) against pccnn_sort_keys, through the C ABI:
bit-exact sorted keys, permutation and gathered points, on two calls in a row, the second with a smaller input,
which runs on the scratch array as the first call left it."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
STATIC_MAX = 1 << 20        # PCCNN_SORT_KEYS_STATIC_MAX of include/pccnn_hip.h


def _both(lib, n, key_bits, seed, with_pts):
    g = torch.Generator(device="cpu").manual_seed(seed)
    keys = torch.randint(0, 1 << key_bits, (n,), generator=g, dtype=torch.int64).to(DEV)
    pts = torch.rand((n, 3), generator=g, dtype=torch.float32).to(DEV) if with_pts else None
    ptr = lambda x: ctypes.c_void_p(x.data_ptr()) if x is not None else ctypes.c_void_p(0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    for static in (False, True):
        # outputs are pre-filled with a pattern so that an element the sort does not write shows up
        skeys = torch.full((n,), -7, dtype=torch.int64, device=DEV)
        perm = torch.full((n,), -7, dtype=torch.int32, device=DEV)
        spts = torch.full((n, 3), -7.0, dtype=torch.float32, device=DEV) if with_pts else None
        if static:
            rc = lib.pccnn_sort_keys_static(ptr(keys), n, key_bits, ptr(skeys), ptr(perm), ptr(pts), 3, ptr(spts),
                                            stream)
        else:
            nbytes = lib.pccnn_sort_keys_workspace_bytes(n)
            ws = torch.empty((nbytes,), dtype=torch.uint8, device=DEV)
            rc = lib.pccnn_sort_keys(ptr(keys), n, key_bits, ptr(skeys), ptr(perm), ptr(pts), 3, ptr(spts), ptr(ws),
                                     nbytes, stream)
        assert rc == 0, lib.pccnn_last_error()
        torch.cuda.synchronize()
        out.append((skeys.cpu().numpy(), perm.cpu().numpy(), None if spts is None else spts.cpu().numpy()))
    (k0, p0, x0), (k1, p1, x1) = out
    host = keys.cpu().numpy()
    assert np.array_equal(p0, np.argsort(host, kind="stable").astype(np.int32))
    assert np.array_equal(k1, k0) and np.array_equal(p1, p0)
    if with_pts:
        assert np.array_equal(x1, x0) and np.array_equal(x0, pts.cpu().numpy()[p0])


def test_static_sort_leaves_the_free_device_memory_unchanged():
    # what the entry point is for: once the first call on the device has looked up the scratch array's address, a
    # call neither allocates nor frees device memory (hipMemGetInfo before and after, inputs and outputs made first)
    from pccnn_lib_amd import _lib
    lib = _lib.load()
    ptr = lambda x: ctypes.c_void_p(0 if x is None else x.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator(device=DEV).manual_seed(9)
    n = 200_000
    keys = torch.randint(0, 1 << 20, (n,), dtype=torch.int64, device=DEV, generator=gen)
    pts = torch.rand((n, 3), device=DEV, generator=gen)
    skeys, perm, spts = torch.empty_like(keys), torch.empty((n,), dtype=torch.int32, device=DEV), torch.empty_like(pts)
    call = lambda count: lib.pccnn_sort_keys_static(ptr(keys), count, 20, ptr(skeys), ptr(perm), ptr(pts), 3, ptr(spts),
                                                   stream)
    assert call(n) == 0, lib.pccnn_last_error()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for count in (n, 50_000, n):
        assert call(count) == 0, lib.pccnn_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(skeys, torch.sort(keys, stable=True)[0])


def test_static_sort_equals_the_workspace_sort_on_two_calls_in_a_row():
    from pccnn_lib_amd import _lib
    lib = _lib.load()
    _both(lib, 300_000, 22, 1, True)        # three passes
    _both(lib, 41_237, 18, 2, True)         # smaller, other digit width and tile size, on the used scratch
    _both(lib, STATIC_MAX, 27, 3, False)    # the largest input it takes
    _both(lib, 1, 5, 4, True)


def test_static_sort_rejects_more_keys_than_its_scratch_holds():
    from pccnn_lib_amd import _lib
    lib = _lib.load()
    n = STATIC_MAX + 1
    keys = torch.zeros((n,), dtype=torch.int64, device=DEV)
    skeys, perm = torch.empty_like(keys), torch.empty((n,), dtype=torch.int32, device=DEV)
    rc = lib.pccnn_sort_keys_static(ctypes.c_void_p(keys.data_ptr()), n, 8, ctypes.c_void_p(skeys.data_ptr()),
                                    ctypes.c_void_p(perm.data_ptr()), ctypes.c_void_p(0), 3, ctypes.c_void_p(0),
                                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -2 and b"at most" in lib.pccnn_last_error()

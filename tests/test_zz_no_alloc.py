"""The entry point that allocates nothing (l2h_argmax_noalloc) against l2h_argmax.

Device memory for its input and output comes from the HIP runtime the library itself is linked to (hipMalloc
through ctypes: plumbing only); the call goes through the C ABI.
Two calls in a row, the second with a smaller input whose answer differs: the array the kernels keep their
intermediate keys in is shared by every call on a GPU and keeps the last call's contents, none of which may
show in the next result.  Bit-exact bar (an index)."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


_HIP = None


def _hip():
    global _HIP
    if _HIP is None:
        _HIP = ctypes.CDLL("libamdhip64.so")  # already mapped by libl2hip.so: the same runtime
        _HIP.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        _HIP.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        _HIP.hipFree.argtypes = [ctypes.c_void_p]
    return _HIP


class _DevMem:
    def __init__(self, nbytes):
        self.p = ctypes.c_void_p()
        assert _hip().hipMalloc(ctypes.byref(self.p), nbytes) == 0

    def put(self, a):
        assert _hip().hipMemcpy(self.p, a.ctypes.data_as(ctypes.c_void_p), a.nbytes, 1) == 0

    def get(self, a):
        assert _hip().hipMemcpy(a.ctypes.data_as(ctypes.c_void_p), self.p, a.nbytes, 2) == 0

    def free(self):
        _hip().hipFree(self.p)


def _noalloc(pkg, ctx, x_host):
    from llama2_jl_amd import _lib
    x, out = _DevMem(x_host.nbytes), _DevMem(4)
    x.put(x_host)
    res = np.array([-7], np.int32)
    out.put(res)  # (synchronous copies: done before the library's stream starts)
    ctx.check(_lib.lib().l2h_argmax_noalloc(ctx.handle, x.p, x_host.size, out.p))
    ctx.sync()
    out.get(res)
    x.free()
    out.free()
    return int(res[0])


def _host(pkg, ctx, x_host):
    from llama2_jl_amd import _lib
    out = ctypes.c_int32(-1)
    ctx.check(_lib.lib().l2h_argmax(ctx.handle, _lib.ptr(x_host), x_host.size, ctypes.byref(out)))
    return out.value


def test_argmax_noalloc_matches_argmax(pkg, ctx):
    from llama2_jl_amd import _lib
    rng = np.random.default_rng(5)
    # first call: 128256 logits, the maximum far out (index 100003), repeated later (first one wins)
    a = rng.standard_normal(128256).astype(np.float32)
    a[100003] = 9.0
    a[120000] = 9.0
    # second call: shorter than the first, its maximum (smaller than 9) at index 17 and again at 4000
    b = rng.standard_normal(5000).astype(np.float32)
    b[17] = 6.5
    b[4000] = 6.5
    for x, want in ((a, 100003), (b, 17)):
        got = _noalloc(pkg, ctx, x)
        assert got == _host(pkg, ctx, x) == want == int(np.argmax(x))
    # all negative, one element, zeros of both signs
    for x in (-np.abs(rng.standard_normal(777)).astype(np.float32) - 1.0, np.array([-3.5], np.float32),
              np.array([-0.0, 0.0, -0.0], np.float32)):
        assert _noalloc(pkg, ctx, x) == _host(pkg, ctx, x) == int(np.argmax(x))
    # sizes beyond the stated maximum, and NULL pointers, are refused
    x, out = _DevMem(16), _DevMem(4)
    for n in (0, -1, (1 << 30) + 1):
        assert _lib.lib().l2h_argmax_noalloc(ctx.handle, x.p, n, out.p) == _lib.EINVAL
    assert _lib.lib().l2h_argmax_noalloc(ctx.handle, None, 4, out.p) == _lib.EINVAL
    assert b"NULL" in _lib.lib().l2h_last_error(ctx.handle)
    x.free()
    out.free()

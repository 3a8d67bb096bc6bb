"""Host-side view of the k-quant super-blocks and the device operators on them.

Mirrors Llama2.jl's src/kquants.jl: the block structs (:7-42) as numpy structured dtypes,
`dequantize` (:49-53) and `vecdot`/`matmul!` (:127-408, src/matmul.jl) as calls into
libl2hip.so.  Nothing here computes on the CPU.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import TYPE_F32, TYPE_Q4_K, TYPE_Q5_K, TYPE_Q6_K

QK_K = 256  # src/kquants.jl:1

block_q4_K = np.dtype([("d", "<f2"), ("dmin", "<f2"), ("scales", "u1", 12), ("qs", "u1", QK_K // 2)])
block_q5_K = np.dtype([("d", "<f2"), ("dmin", "<f2"), ("scales", "u1", 12), ("qh", "u1", QK_K // 8),
                       ("qs", "u1", QK_K // 2)])
block_q6_K = np.dtype([("ql", "u1", QK_K // 2), ("qh", "u1", QK_K // 4), ("scales", "i1", QK_K // 16), ("d", "<f2")])
block_q8_K = np.dtype([("d", "<f4"), ("qs", "i1", QK_K), ("bsums", "<i2", QK_K // 16)])

BLOCK_DTYPE = {TYPE_Q4_K: block_q4_K, TYPE_Q5_K: block_q5_K, TYPE_Q6_K: block_q6_K}
BLOCK_BYTES = {TYPE_F32: 4, TYPE_Q4_K: 144, TYPE_Q5_K: 176, TYPE_Q6_K: 210}
TYPE_NAME = {TYPE_F32: "F32", TYPE_Q4_K: "Q4_K", TYPE_Q5_K: "Q5_K", TYPE_Q6_K: "Q6_K"}
assert block_q4_K.itemsize == 144 and block_q5_K.itemsize == 176
assert block_q6_K.itemsize == 210 and block_q8_K.itemsize == 292


class QuantMatrix:
    """A k-quant weight matrix on the host: `ne1` output rows of `ne0` input features, each row
    `ne0/256` consecutive super-blocks -- Julia's Array{block_T}(ne0/256, ne1)
    (src/load_gguf.jl:141-151).  `data` is a uint8 array (possibly a memory map) of the raw
    GGUF bytes."""

    def __init__(self, ggml_type, data, ne0, ne1):
        if ggml_type not in BLOCK_DTYPE:
            raise ValueError("tensor type %r not implemented" % (ggml_type,))  # load_gguf.jl:153
        if ne0 % QK_K != 0:
            raise ValueError("ne0 = %d is not a multiple of %d" % (ne0, QK_K))  # load_gguf.jl:141
        data = np.asarray(data).reshape(-1).view(np.uint8)
        expect = (ne0 // QK_K) * ne1 * BLOCK_BYTES[ggml_type]
        if data.size != expect:
            raise ValueError("expected %d bytes of blocks, got %d" % (expect, data.size))
        self.type, self.data, self.ne0, self.ne1 = ggml_type, data, ne0, ne1

    @property
    def shape(self):  # (in_features, out_features), as size(A) of the Julia matrix times 256
        return (self.ne0, self.ne1)

    @property
    def blocks(self):
        return self.data.view(BLOCK_DTYPE[self.type]).reshape(self.ne1, self.ne0 // QK_K)

    def rows(self, start, stop):
        """view(A, :, start:stop) (0-based, stop exclusive): a contiguous range of output rows,
        as used for Phi-3's fused tensors (src/load_gguf.jl:264-276)."""
        rb = (self.ne0 // QK_K) * BLOCK_BYTES[self.type]
        return QuantMatrix(self.type, self.data[start * rb:stop * rb], self.ne0, stop - start)

    def row_bytes(self, i):
        rb = (self.ne0 // QK_K) * BLOCK_BYTES[self.type]
        return self.data[i * rb:(i + 1) * rb]


def matrix_type(A):
    return A.type if isinstance(A, QuantMatrix) else TYPE_F32


def matrix_shape(A):
    """(ne0, ne1) = (input features, output rows)."""
    if isinstance(A, QuantMatrix):
        return A.ne0, A.ne1
    return A.shape[1], A.shape[0]


def matrix_bytes(A):
    if isinstance(A, QuantMatrix):
        return np.ascontiguousarray(A.data)
    return np.ascontiguousarray(A, dtype=np.float32)


def dequantize(x, ggml_type=None, ctx=None):
    """dequantize(x) (src/kquants.jl:49-53) on the device.  x: QuantMatrix (all rows, row-major
    output), or raw block bytes with an explicit ggml_type."""
    ctx = ctx or _lib.default_context()
    if isinstance(x, QuantMatrix):
        ggml_type, raw = x.type, np.ascontiguousarray(x.data)
    else:
        raw = np.ascontiguousarray(np.asarray(x).reshape(-1).view(np.uint8))
    if ggml_type == TYPE_F32:
        nb = raw.size // 4
        out = np.empty(nb, np.float32)
    else:
        nb = raw.size // BLOCK_BYTES[ggml_type]
        out = np.empty(nb * QK_K, np.float32)
    ctx.check(_lib.lib().l2h_dequantize(ctx.handle, ggml_type, _lib.ptr(raw), nb, _lib.ptr(out)))
    return out


def quantize_q8_K(x, ctx=None):
    """q8_K image of a float vector: array of block_q8_K records (src/kquants.jl:37-42)."""
    ctx = ctx or _lib.default_context()
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros(x.size // QK_K, block_q8_K)
    ctx.check(_lib.lib().l2h_quantize_q8k(ctx.handle, _lib.ptr(x), x.size, _lib.ptr(out)))
    return out


def matmul(A, x, return_ints=False, ctx=None):
    """matmul!(y, A, x): y = A' x (src/matmul.jl:3-23).  A: QuantMatrix or float32 array of
    shape (out, in).  With return_ints also returns the per-(row, super-block) integer sums
    (I_sc, I_min) the k-quant kernel formed."""
    ctx = ctx or _lib.default_context()
    ne0, ne1 = matrix_shape(A)
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.size != ne0:
        raise ValueError("x has %d elements, A expects %d" % (x.size, ne0))
    y = np.empty(ne1, np.float32)
    isc = imin = None
    if return_ints:
        isc = np.zeros((ne1, ne0 // QK_K), np.int32)
        imin = np.zeros((ne1, ne0 // QK_K), np.int32)
    raw = matrix_bytes(A)
    ctx.check(_lib.lib().l2h_matmul(ctx.handle, matrix_type(A), _lib.ptr(raw), ne0, ne1, _lib.ptr(x), _lib.ptr(y),
                                    _lib.ptr(isc), _lib.ptr(imin)))
    return (y, isc, imin) if return_ints else y


def quantize_weights(x, ggml_type, nthreads=0):
    """fp32 -> k-quant super-blocks (host code in the library; the reference has no encoder).
    x: (out, in) float32.  Returns a QuantMatrix."""
    import os
    x = np.ascontiguousarray(x, dtype=np.float32)
    ne1, ne0 = x.shape
    out = np.empty((ne0 // QK_K) * ne1 * BLOCK_BYTES[ggml_type], np.uint8)
    rc = _lib.lib().l2h_quantize_weights(ggml_type, _lib.ptr(x), x.size, _lib.ptr(out),
                                         nthreads or min(16, os.cpu_count() or 1))
    if rc != 0:
        raise _lib.L2HError(rc, "l2h_quantize_weights failed")
    return QuantMatrix(ggml_type, out, ne0, ne1)

"""ctypes binding of libl2hip.so (the C ABI declared in include/l2h.h).

The library is the only compute path: if it is missing this module raises, it never
falls back to a CPU implementation.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# L2H_LIB names another build of the same library (e.g. the profiling build libl2hip_tl.so)
LIB_PATH = os.environ.get("L2H_LIB") or os.path.join(HERE, "libl2hip.so")

# error codes / enums of include/l2h.h
OK, EINVAL, ETYPE, ESTATE, EHIP, ENOMEM, ENODEV = 0, -1, -2, -3, -4, -5, -6
TYPE_F32, TYPE_Q4_K, TYPE_Q5_K, TYPE_Q6_K = 0, 12, 13, 14
(TOK_EMB, RMS_FINAL, OUTPUT, RMS_ATT, RMS_FFN, WQ, WK, WV, WO, W1, W2, W3) = range(12)
N_ROLES = 12


class L2HError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("l2h error %d: %s" % (code, msg))
        self.code = code


class Config(C.Structure):
    _fields_ = [
        ("dim", C.c_int32), ("hidden_dim", C.c_int32), ("n_layers", C.c_int32), ("n_heads", C.c_int32),
        ("n_kv_heads", C.c_int32), ("vocab_size", C.c_int32), ("seq_len", C.c_int32),
        ("rope_freq_base", C.c_float), ("rope_is_neox", C.c_int32),
    ]


_P = C.c_void_p
_I, _I64, _F = C.c_int, C.c_int64, C.c_float
_PF, _PI32 = C.POINTER(C.c_float), C.POINTER(C.c_int32)

# name -> (restype, argtypes); every symbol include/l2h.h declares
SIGNATURES = {
    "l2h_ctx_create": (_I, [_I, C.POINTER(_P)]),
    "l2h_ctx_destroy": (None, [_P]),
    "l2h_last_error": (C.c_char_p, [_P]),
    "l2h_sync": (_I, [_P]),
    "l2h_device_info": (_I, [_P, C.c_char_p, _I, _PI32, C.POINTER(_I64)]),
    "l2h_model_create": (_I, [_P, C.POINTER(Config), C.POINTER(_P)]),
    "l2h_model_destroy": (None, [_P]),
    "l2h_model_set_tensor": (_I, [_P, _I, _I, _I, _P, _I64, _I64]),
    "l2h_model_get_tensor": (_I, [_P, _I, _I, _P, _I64]),
    "l2h_model_set_kv_type": (_I, [_P, _I]),
    "l2h_model_path_reason": (C.c_char_p, [_P]),
    "l2h_model_set_path": (_I, [_P, _I]),
    "l2h_model_set_wait_limit": (_I, [_P, C.c_uint]),
    "l2h_model_set_prefill_copy": (_I, [_P, _I]),
    "l2h_model_set_prefill_library": (_I, [_P, _I]),
    "l2h_model_prefill_library": (_I, [_P]),
    "l2h_model_path": (_I, [_P]),
    "l2h_model_steps_per_launch": (_I, [_P]),
    "l2h_model_finalize": (_I, [_P]),
    "l2h_state_reset": (_I, [_P]),
    "l2h_kv_write": (_I, [_P, _I, _I, _I, _P, _P]),
    "l2h_kv_read": (_I, [_P, _I, _I, _I, _P, _P]),
    "l2h_forward": (_I, [_P, _I, _I, _P, _PI32]),
    "l2h_generate_greedy": (_I, [_P, _P, _I, _I, _I, _P, _P]),
    "l2h_generate_greedy_timed": (_I, [_P, _P, _I, _I, _I, _P, _PF]),
    "l2h_prefill": (_I, [_P, _P, _I, _I, _P, _PI32]),
    "l2h_sample": (_I, [_P, C.c_float, C.c_float, _PI32, _P]),
    "l2h_state_read": (_I, [_P, _I, _P, _I64]),
    "l2h_quantize_q8k": (_I, [_P, _P, _I64, _P]),
    "l2h_dequantize": (_I, [_P, _I, _P, _I64, _P]),
    "l2h_matmul": (_I, [_P, _I, _P, _I64, _I64, _P, _P, _P, _P]),
    "l2h_model_matmul": (_I, [_P, _I, _I, _P, _P]),
    "l2h_rmsnorm": (_I, [_P, _P, _P, _P, _I64]),
    "l2h_rmsnorm_q8k": (_I, [_P, _P, _P, _I64, _P]),
    "l2h_rope": (_I, [_P, _P, _I, _I, _I, _F, _I]),
    "l2h_softmax": (_I, [_P, _P, _I64]),
    "l2h_attention": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I]),
    "l2h_swiglu": (_I, [_P, _P, _P, _I64]),
    "l2h_argmax": (_I, [_P, _P, _I64, _PI32]),
    "l2h_argmax_noalloc": (_I, [_P, _P, _I64, _P]),
    "l2h_profile_matvec": (_I, [_P, _I, _I, _PF, C.POINTER(_I64)]),
    "l2h_profile_stream_read": (_I, [_P, _I64, _I, _PF]),
    "l2h_synth_normal": (_I, [C.c_uint64, C.c_uint64, _I64, _I64, _F, _P, _I]),
    "l2h_quantize_weights": (_I, [_I, _P, _I64, _P, _I]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python llama2.jl_amd/build.py` (needs hipcc). "
                "There is no CPU fallback." % LIB_PATH)
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def ptr(a):
    """void* of a C-contiguous numpy array (or None)."""
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


class Context:
    """l2h_ctx: one HIP device + stream.  A process-wide default is kept by default_context()."""

    def __init__(self, device=0):
        self.handle = _P()
        rc = lib().l2h_ctx_create(device, C.byref(self.handle))
        if rc != OK:
            raise L2HError(rc, lib().l2h_last_error(None).decode())

    def check(self, rc):
        if rc != OK:
            raise L2HError(rc, lib().l2h_last_error(self.handle).decode())

    def device_info(self):
        name = C.create_string_buffer(256)
        ncu, mem = C.c_int32(), _I64()
        self.check(lib().l2h_device_info(self.handle, name, 256, C.byref(ncu), C.byref(mem)))
        return {"name": name.value.decode(), "n_cu": ncu.value, "hbm_bytes": mem.value}

    def sync(self):
        self.check(lib().l2h_sync(self.handle))

    def close(self):
        if self.handle:
            lib().l2h_ctx_destroy(self.handle)
            self.handle = _P()


_default_ctx = None


def default_context():
    global _default_ctx
    if _default_ctx is None:
        _default_ctx = Context(int(os.environ.get("L2H_DEVICE", "0")))
    return _default_ctx

"""ctypes wrapper of oracle/libl2c.so, the CPU restatement of the reference (see l2c.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, never by the product package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libl2c.so")

ACT_Q8K, CANON, KV16 = 1, 2, 4
GPU_SPEC = ACT_Q8K | CANON  # the mode the HIP path implements
REFERENCE = 0               # float activations, fp32 sums in index order: the reference snapshot

F32, Q4_K, Q5_K, Q6_K = 0, 12, 13, 14
BLOCK_BYTES = {F32: 4, Q4_K: 144, Q5_K: 176, Q6_K: 210}
(TOK_EMB, RMS_FINAL, OUTPUT, RMS_ATT, RMS_FFN, WQ, WK, WV, WO, W1, W2, W3) = range(12)

block_q8_K = np.dtype([("d", "<f4"), ("qs", "i1", 256), ("bsums", "<i2", 16)])


def build(force=False):
    src = os.path.join(HERE, "l2c.c")
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(src):
        subprocess.run(["make", "-C", HERE, "-B", "libl2c.so"], check=True, capture_output=True)
    return LIB_PATH


class Config(C.Structure):
    _fields_ = [("dim", C.c_int32), ("hidden_dim", C.c_int32), ("n_layers", C.c_int32), ("n_heads", C.c_int32),
                ("n_kv_heads", C.c_int32), ("vocab_size", C.c_int32), ("seq_len", C.c_int32),
                ("rope_freq_base", C.c_float), ("rope_is_neox", C.c_int32)]


_lib = None
_P, _I, _I64, _F = C.c_void_p, C.c_int, C.c_int64, C.c_float


def lib():
    global _lib
    if _lib is None:
        build()
        l = C.CDLL(LIB_PATH)
        sig = {
            "l2c_block_bytes": (_I64, [_I]),
            "l2c_fp16_to_fp32": (_F, [C.c_uint16]),
            "l2c_fp32_to_fp16": (C.c_uint16, [_F]),
            "l2c_scale_min_k4": (None, [_P, _P, _P]),
            "l2c_dequantize": (_I, [_I, _P, _I64, _P]),
            "l2c_vecdot_f32act": (_F, [_I, _P, _I64, _P, _I]),
            "l2c_quantize_q8_K": (None, [_P, _I64, _P]),
            "l2c_vecdot_q8k": (_F, [_I, _P, _P, _I64, _I, _P, _P]),
            "l2c_matmul": (_I, [_I, _P, _I64, _I64, _P, _P, _P, _I, _I]),
            "l2c_rmsnorm": (None, [_P, _P, _P, _I64, _I]),
            "l2c_rope_theta_scale": (_F, [_F, _I]),
            "l2c_rope": (None, [_P, _I, _I, _I, _F, _I, _I]),
            "l2c_softmax": (None, [_P, _I64, _I]),
            "l2c_attention": (None, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I]),
            "l2c_swiglu": (None, [_P, _P, _I64, _I]),
            "l2c_argmax": (_I64, [_P, _I64]),
            "l2c_model_create": (_P, [C.POINTER(Config), _I]),
            "l2c_model_destroy": (None, [_P]),
            "l2c_model_set_tensor": (_I, [_P, _I, _I, _I, _P, _I64, _I64]),
            "l2c_state_reset": (None, [_P]),
            "l2c_kv_write": (_I, [_P, _I, _I, _I, _P, _P]),
            "l2c_kv_read": (_I, [_P, _I, _I, _I, _P, _P]),
            "l2c_forward": (_I, [_P, _I, _I, _I, _P]),
            "l2c_generate_greedy": (_I, [_P, _P, _I, _I, _I, _I, _P, _P]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(l, name)
            fn.restype, fn.argtypes = res, args
        _lib = l
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _raw(a):
    return np.ascontiguousarray(np.asarray(a).reshape(-1).view(np.uint8))


def dequantize(typ, blocks):
    raw = _raw(blocks)
    nb = raw.size // BLOCK_BYTES[typ]
    y = np.empty(nb if typ == F32 else nb * 256, np.float32)
    assert lib().l2c_dequantize(typ, _p(raw), nb, _p(y)) == 0
    return y


def quantize_q8_K(x):
    x = _f32(x)
    out = np.zeros(x.size // 256, block_q8_K)
    lib().l2c_quantize_q8_K(_p(x), x.size, _p(out))
    return out


def vecdot_f32act(typ, row_blocks, y, canon=0):
    raw, y = _raw(row_blocks), _f32(y)
    return float(lib().l2c_vecdot_f32act(typ, _p(raw), raw.size // BLOCK_BYTES[typ], _p(y), canon))


def vecdot_q8k(typ, row_blocks, q8, canon=1):
    raw = _raw(row_blocks)
    nb = raw.size // BLOCK_BYTES[typ]
    q8 = np.ascontiguousarray(q8)
    isc, imin = np.zeros(nb, np.int32), np.zeros(nb, np.int32)
    v = float(lib().l2c_vecdot_q8k(typ, _p(raw), _p(q8), nb, canon, _p(isc), _p(imin)))
    return v, isc, imin


def matmul(typ, A, ne0, ne1, x, mode, nthreads=1):
    raw, x = _raw(A), _f32(x)
    y = np.empty(ne1, np.float32)
    assert lib().l2c_matmul(typ, _p(raw), ne0, ne1, _p(x), None, _p(y), mode, nthreads) == 0
    return y


def matmul_ints(typ, A, ne0, ne1, x):
    """per-(row, block) integer sums of the q8_K path, via vecdot_q8k row by row"""
    raw = _raw(A)
    q8 = quantize_q8_K(x)
    nb = ne0 // 256
    rb = nb * BLOCK_BYTES[typ]
    isc, imin = np.zeros((ne1, nb), np.int32), np.zeros((ne1, nb), np.int32)
    for i in range(ne1):
        _, isc[i], imin[i] = vecdot_q8k(typ, raw[i * rb:(i + 1) * rb], q8)
    return isc, imin


def rmsnorm(x, w, mode):
    x, w = _f32(x), _f32(w)
    o = np.empty_like(x)
    lib().l2c_rmsnorm(_p(o), _p(x), _p(w), x.size, mode)
    return o


def rope(x, head_size, n_heads, pos0, freq_base, neox, mode):
    x = _f32(x).copy()
    ts = lib().l2c_rope_theta_scale(freq_base, head_size)
    lib().l2c_rope(_p(x), head_size, n_heads, pos0, ts, int(neox), mode)
    return x


def softmax(x, mode):
    x = _f32(x).copy()
    lib().l2c_softmax(_p(x), x.size, mode)
    return x


def attention(q, kc, vc, head_size, n_heads, n_kv_heads, pos0, mode):
    q, kc, vc = _f32(q), _f32(kc), _f32(vc)
    out = np.empty(head_size * n_heads, np.float32)
    att = np.empty(n_heads * (pos0 + 1), np.float32)
    lib().l2c_attention(_p(out), _p(q), _p(kc), _p(vc), _p(att), head_size, n_heads, n_kv_heads, pos0, mode)
    return out, att.reshape(n_heads, pos0 + 1)


def swiglu(hb, hb2, mode):
    hb, hb2 = _f32(hb).copy(), _f32(hb2)
    lib().l2c_swiglu(_p(hb), _p(hb2), hb.size, mode)
    return hb


def argmax(x):
    x = _f32(x)
    return int(lib().l2c_argmax(_p(x), x.size))


class Model:
    """l2c_model over host tensors given as (ggml_type, uint8/float32 array, ne0, ne1)."""

    def __init__(self, cfg, tensors, nthreads=1):
        """cfg: dict or object with the ModelConfig fields; tensors: {(role, layer): (type, array, ne0, ne1)}"""
        g = (lambda k: cfg[k]) if isinstance(cfg, dict) else (lambda k: getattr(cfg, k))
        self.cfg = Config(g("dim"), g("hidden_dim"), g("n_layers"), g("n_heads"), g("n_kv_heads"), g("vocab_size"),
                          g("seq_len"), float(g("rope_freq_base")), int(bool(g("rope_is_neox"))))
        self.h = lib().l2c_model_create(C.byref(self.cfg), nthreads)
        self._keep = []
        for (role, layer), (typ, arr, ne0, ne1) in tensors.items():
            a = np.ascontiguousarray(arr)
            self._keep.append(a)
            assert lib().l2c_model_set_tensor(self.h, role, layer, typ, _p(a), ne0, ne1) == 0

    def reset(self):
        lib().l2c_state_reset(self.h)

    def forward(self, token, pos0, mode):
        logits = np.empty(self.cfg.vocab_size, np.float32)
        rc = lib().l2c_forward(self.h, token, pos0, mode, _p(logits))
        assert rc == 0, rc
        return logits

    def generate_greedy(self, prompt, n_new, mode, pos0=0):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.zeros(max(n_new, 1), np.int32)
        logits = np.empty(self.cfg.vocab_size, np.float32)
        n = lib().l2c_generate_greedy(self.h, _p(prompt), prompt.size, pos0, n_new, mode, _p(out), _p(logits))
        assert n >= 0, n
        return out[:n], logits

    def kv_write(self, layer, pos0, k, v):
        k, v = _f32(k), _f32(v)
        assert lib().l2c_kv_write(self.h, layer, pos0, k.shape[0], _p(k), _p(v)) == 0

    def kv_read(self, layer, pos0, n):
        kv_dim = self.cfg.dim // self.cfg.n_heads * self.cfg.n_kv_heads
        k, v = np.empty((n, kv_dim), np.float32), np.empty((n, kv_dim), np.float32)
        assert lib().l2c_kv_read(self.h, layer, pos0, n, _p(k), _p(v)) == 0
        return k, v

    def close(self):
        if self.h:
            lib().l2c_model_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()


def model_from_language_model(lm, nthreads=1):
    """Builds the oracle model from a host-side LanguageModel of the product package (duck-typed:
    only attributes are read, so the oracle does not import the package)."""
    w, c = lm.weights, lm.config
    tensors = {}

    def put(role, layer, A):
        if hasattr(A, "type") and hasattr(A, "ne0"):  # QuantMatrix
            tensors[(role, layer)] = (A.type, A.data, A.ne0, A.ne1)
        else:
            a = np.ascontiguousarray(A, dtype=np.float32)
            if a.ndim == 1:
                tensors[(role, layer)] = (F32, a, a.size, 1)
            else:
                tensors[(role, layer)] = (F32, a, a.shape[1], a.shape[0])

    put(TOK_EMB, 0, w.token_embedding_table)
    put(RMS_FINAL, 0, w.rms_final_weight)
    put(OUTPUT, 0, w.output_weight)
    for l, lw in enumerate(w.layers):
        for name, role in (("rms_att_weight", RMS_ATT), ("rms_ffn_weight", RMS_FFN), ("wq", WQ), ("wk", WK),
                           ("wv", WV), ("wo", WO), ("w1", W1), ("w2", W2), ("w3", W3)):
            put(role, l, getattr(lw, name))
    return Model(c, tensors, nthreads)

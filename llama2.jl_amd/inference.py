"""Model containers and the decode loop of Llama2.jl (src/inference.jl), bound to the HIP library.

Same names and argument meaning as the reference (ModelConfig, TransformerLayerWeights,
TransformerWeights, LanguageModel, RunState, transformer!, sample); token ids and positions
are 0-based in Python.  Weights live on the host as the loaders produce them and are uploaded
once, on first use, into the device layout; all arithmetic runs in libl2hip.so.
"""
import ctypes as C
import sys
import time
from dataclasses import dataclass, field
from typing import Any, List

import numpy as np

from . import _lib
from .kquants import matrix_bytes, matrix_shape, matrix_type
from .tokenizer import encode, token_bytes


@dataclass
class ModelConfig:  # src/inference.jl:1-11
    dim: int
    hidden_dim: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    vocab_size: int
    seq_len: int
    rope_freq_base: float = 10000.0
    rope_is_neox: bool = False

    def __str__(self):  # src/inference.jl:13-25
        rows = ["dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len", "rope_freq_base",
                "rope_is_neox"]
        return "ModelConfig(\n" + "".join("  %-14s = %s,\n" % (r, getattr(self, r)) for r in rows) + ")"


@dataclass
class TransformerLayerWeights:  # src/inference.jl:27-40; matrices are float32 (out, in) arrays or QuantMatrix
    rms_att_weight: np.ndarray
    rms_ffn_weight: np.ndarray
    wq: Any
    wk: Any
    wv: Any
    wo: Any
    w1: Any
    w2: Any
    w3: Any


@dataclass
class TransformerWeights:  # src/inference.jl:42-48
    token_embedding_table: Any
    layers: List[TransformerLayerWeights]
    rms_final_weight: np.ndarray
    output_weight: Any


_LAYER_ROLES = [("rms_att_weight", _lib.RMS_ATT), ("rms_ffn_weight", _lib.RMS_FFN), ("wq", _lib.WQ), ("wk", _lib.WK),
                ("wv", _lib.WV), ("wo", _lib.WO), ("w1", _lib.W1), ("w2", _lib.W2), ("w3", _lib.W3)]


class DeviceModel:
    """l2h_model: the weights in HBM plus the RunState (activations, KV cache)."""

    def __init__(self, config, weights, ctx=None, path=0, kv_fp16=False):
        self.ctx = ctx or _lib.default_context()
        self.config = config
        cfg = _lib.Config(config.dim, config.hidden_dim, config.n_layers, config.n_heads, config.n_kv_heads,
                          config.vocab_size, config.seq_len, float(config.rope_freq_base),
                          1 if config.rope_is_neox else 0)
        self.handle = C.c_void_p()
        self._shapes = {}
        self.ctx.check(_lib.lib().l2h_model_create(self.ctx.handle, C.byref(cfg), C.byref(self.handle)))
        try:
            self._set(_lib.TOK_EMB, 0, weights.token_embedding_table)
            self._set(_lib.RMS_FINAL, 0, weights.rms_final_weight)
            self._set(_lib.OUTPUT, 0, weights.output_weight)
            if len(weights.layers) != config.n_layers:
                raise ValueError("config.n_layers = %d but %d layers given" % (config.n_layers, len(weights.layers)))
            for l, lw in enumerate(weights.layers):
                for name, role in _LAYER_ROLES:
                    self._set(role, l, getattr(lw, name))
            if kv_fp16:
                self.ctx.check(_lib.lib().l2h_model_set_kv_type(self.handle, 1))
            self.ctx.check(_lib.lib().l2h_model_set_path(self.handle, path))
            self.ctx.check(_lib.lib().l2h_model_finalize(self.handle))
            self.path = _lib.lib().l2h_model_path(self.handle)  # 1 = kernel per phase, 2 = persistent kernel, 3 = streaming
            self.path_reason = _lib.lib().l2h_model_path_reason(self.handle).decode()  # why not 3 ("" if 3)
            self.steps_per_launch = _lib.lib().l2h_model_steps_per_launch(self.handle)  # token-loop steps per kernel launch
        except Exception:
            self.close()
            raise

    def _set(self, role, layer, A):
        if isinstance(A, np.ndarray) and A.ndim == 1:
            ne0, ne1, typ, raw = A.size, 1, _lib.TYPE_F32, np.ascontiguousarray(A, dtype=np.float32)
        else:
            (ne0, ne1), typ, raw = matrix_shape(A), matrix_type(A), matrix_bytes(A)
        self.ctx.check(_lib.lib().l2h_model_set_tensor(self.handle, role, layer, typ, _lib.ptr(raw), ne0, ne1))
        self._shapes[(role, layer)] = (ne0, ne1)

    def close(self):
        if self.handle:
            _lib.lib().l2h_model_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # --- RunState operations ---
    def reset(self):
        self.ctx.check(_lib.lib().l2h_state_reset(self.handle))

    def matmul(self, role, layer, x):
        """matmul!(y, A, x) with A the resident matrix `role` of `layer` (l2h_model_matmul): the seam at which the
        reference's own transformer! can run on device-resident weights."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        ne0, ne1 = self._shapes[(role, 0 if role < 3 else layer)]
        if x.size != ne0:
            raise ValueError("x has %d elements, the matrix expects %d" % (x.size, ne0))
        y = np.empty(ne1, np.float32)
        self.ctx.check(_lib.lib().l2h_model_matmul(self.handle, role, layer, _lib.ptr(x), _lib.ptr(y)))
        return y

    def set_wait_limit(self, spins):
        """Bound of the streaming kernel's device-side waits (l2h_model_set_wait_limit)."""
        self.ctx.check(_lib.lib().l2h_model_set_wait_limit(self.handle, int(spins)))

    def set_prefill_copy(self, on):
        """Whether prefill multiplies from a resident bf16 copy of the weights (l2h_model_set_prefill_copy)."""
        self.ctx.check(_lib.lib().l2h_model_set_prefill_copy(self.handle, 1 if on else 0))

    def set_prefill_library(self, on):
        """Whether prefill runs its plain products (q|k|v, wo, w2) through hipBLASLt (l2h_model_set_prefill_library)."""
        self.ctx.check(_lib.lib().l2h_model_set_prefill_library(self.handle, 1 if on else 0))

    @property
    def prefill_library(self):
        """True if the last prefill ran those products through hipBLASLt (l2h_model_prefill_library)."""
        return bool(_lib.lib().l2h_model_prefill_library(self.handle))

    def forward(self, token, pos, want_logits=True):
        """transformer!(token, pos, ...) (src/inference.jl:222-315): returns (logits, argmax)."""
        logits = np.empty(self.config.vocab_size, np.float32) if want_logits else None
        am = C.c_int32()
        self.ctx.check(_lib.lib().l2h_forward(self.handle, int(token), int(pos), _lib.ptr(logits), C.byref(am)))
        return logits, am.value

    def generate_greedy(self, prompt, n_new, pos0=0, want_logits=False, timed=False):
        """Greedy token loop on the device (src/inference.jl:349-386 at temperature 0)."""
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.zeros(max(n_new, 1), np.int32)
        if timed:
            ms = C.c_float()
            self.ctx.check(_lib.lib().l2h_generate_greedy_timed(self.handle, _lib.ptr(prompt), prompt.size, pos0, n_new,
                                                                _lib.ptr(out), C.byref(ms)))
            return out[:n_new], ms.value
        logits = np.empty(self.config.vocab_size, np.float32) if want_logits else None
        self.ctx.check(_lib.lib().l2h_generate_greedy(self.handle, _lib.ptr(prompt), prompt.size, pos0, n_new,
                                                      _lib.ptr(out), _lib.ptr(logits)))
        return (out[:n_new], logits) if want_logits else out[:n_new]

    def prefill(self, tokens, pos0=0, want_logits=True):
        """Batched prompt pass over positions pos0..pos0+len(tokens)-1: fills the K/V cache and returns
        (logits of the last position, their argmax) like calling forward() for each position in turn
        (src/inference.jl:222-315), with the matrix products in bf16 on the matrix cores."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.empty(self.config.vocab_size, np.float32) if want_logits else None
        nxt = C.c_int32()
        self.ctx.check(_lib.lib().l2h_prefill(self.handle, _lib.ptr(tokens), tokens.size, int(pos0), _lib.ptr(logits),
                                              C.byref(nxt)))
        return logits, nxt.value

    def sample_token(self, temperature, u, want_probs=False):
        """Temperature sampling from the logits of the last step (src/inference.jl:363-367) with the
        uniform number u in [0, 1) standing in for wsample's draw."""
        probs = np.empty(self.config.vocab_size, np.float32) if want_probs else None
        tok = C.c_int32()
        self.ctx.check(_lib.lib().l2h_sample(self.handle, float(temperature), float(u), C.byref(tok), _lib.ptr(probs)))
        return (tok.value, probs) if want_probs else tok.value

    def kv_write(self, layer, pos0, k, v):
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        self.ctx.check(_lib.lib().l2h_kv_write(self.handle, layer, pos0, k.shape[0], _lib.ptr(k), _lib.ptr(v)))

    def kv_read(self, layer, pos0, n):
        kv_dim = self.config.dim // self.config.n_heads * self.config.n_kv_heads
        k = np.empty((n, kv_dim), np.float32)
        v = np.empty((n, kv_dim), np.float32)
        self.ctx.check(_lib.lib().l2h_kv_read(self.handle, layer, pos0, n, _lib.ptr(k), _lib.ptr(v)))
        return k, v

    def get_tensor(self, role, layer, nbytes):
        out = np.empty(nbytes, np.uint8)
        self.ctx.check(_lib.lib().l2h_model_get_tensor(self.handle, role, layer, _lib.ptr(out), nbytes))
        return out

    _STATE = {"x": 0, "xb": 1, "q": 2, "hb": 5, "logits": 6}

    def state(self, name):
        c = self.config
        kv_dim = c.dim // c.n_heads * c.n_kv_heads
        n = {"x": c.dim, "xb": c.dim, "q": c.dim, "hb": c.hidden_dim, "logits": c.vocab_size}[name]
        out = np.empty(n, np.float32)
        self.ctx.check(_lib.lib().l2h_state_read(self.handle, self._STATE[name], _lib.ptr(out), n))
        return out

    def profile_matvec(self, role, iters=20):
        us, b = C.c_float(), C.c_int64()
        self.ctx.check(_lib.lib().l2h_profile_matvec(self.handle, role, iters, C.byref(us), C.byref(b)))
        return us.value, b.value


class LanguageModel:  # src/inference.jl:50-54
    def __init__(self, config, tokenizer, weights):
        self.config, self.tokenizer, self.weights = config, tokenizer, weights
        self._device = None

    def device(self, ctx=None, path=0, kv_fp16=False):
        """Upload once; later calls reuse the resident copy (a closed one is replaced).  path: see
        l2h_model_set_path; kv_fp16: an fp16 KV cache (l2h_model_set_kv_type).  Both take effect when the copy is made."""
        if self._device is None or not self._device.handle:
            self._device = DeviceModel(self.config, self.weights, ctx, path, kv_fp16)
        return self._device

    def __str__(self):  # src/inference.jl:56-60
        return "LanguageModel(\n%s)" % self.config


class RunState:
    """RunState(config) (src/inference.jl:72-100): a fresh, zeroed KV cache on the device model."""

    def __init__(self, model):
        self.dev = model.device()
        self.dev.reset()
        self.logits = None


def transformer_(token, pos, config, s, weights=None):
    """transformer!(token, pos, config, s, weights) (src/inference.jl:222): forwards one token at
    0-based position pos and leaves the logits in s.logits."""
    s.logits, _ = s.dev.forward(token, pos)
    return None


def generate(model, prompt_tokens, n_new, pos0=0, want_logits=False):
    """Greedy continuation of token ids; the prompts of the benchmark configurations are ids, which
    the reference's sample() cannot take (it accepts a String only, src/inference.jl:319)."""
    s = RunState(model)
    return s.dev.generate_greedy(prompt_tokens, n_new, pos0, want_logits=want_logits)


def sample(model, prompt="", temperature=0.9, stop_on_special_token=True, max_seq_len=None, bos_token=True,
           rng=None, out=None):
    """sample(model, prompt; temperature, stop_on_special_token, max_seq_len, bos_token)
    (src/inference.jl:317-395): prints the continuation and the achieved tok/s; returns None."""
    out = out or sys.stdout
    if not bos_token and len(prompt) == 0:
        raise ValueError("Prompt cannot be empty if bos_token = false")  # :326-328
    config, tokenizer = model.config, model.tokenizer
    prompt_tokens = encode(prompt, tokenizer)  # :332
    state = RunState(model)  # :334
    time_start = time.perf_counter()
    if bos_token:
        prompt_tokens.insert(0, tokenizer.bos_token_id)  # :338-340
    else:
        _emit(out, token_bytes(tokenizer, prompt_tokens[0]))  # :342-344
    limit = config.seq_len if max_seq_len is None else min(config.seq_len, max_seq_len)  # :349
    rng = rng or np.random.default_rng()
    token = prompt_tokens[0]
    generated_seq_len = 0
    special = (tokenizer.bos_token_id, tokenizer.eos_token_id)
    pos = 0
    while pos < limit:
        if temperature == 0.0 and pos + 1 >= len(prompt_tokens):
            # greedy tail: run a burst of steps on the device, then scan it for a stop token
            burst = min(32, limit - pos)
            ids = state.dev.generate_greedy([token], burst, pos0=pos)
            stop = False
            for nxt in ids:
                generated_seq_len += 1
                pos += 1
                if stop_on_special_token and nxt in special:  # :371-373
                    stop = True
                    break
                _emit(out, token_bytes(tokenizer, nxt))
                token = int(nxt)
            if stop:
                break
            continue
        logits, am = state.dev.forward(token, pos, want_logits=False)  # :351
        generated_seq_len += 1
        if pos + 1 < len(prompt_tokens):
            nxt = prompt_tokens[pos + 1]  # :354-355
        elif temperature == 0.0:
            nxt = am  # :360
        else:
            # logits ./= temperature; softmax!; wsample (:363-367) on the device, the draw from this rng
            nxt = state.dev.sample_token(temperature, min(float(rng.random()), 0.99999994))
        pos += 1
        if stop_on_special_token and nxt in special:
            break
        _emit(out, token_bytes(tokenizer, nxt))  # :375-382
        token = nxt  # :385
    out.write("\n")
    elapsed = time.perf_counter() - time_start
    out.write("-------\nachieved tok/s: %.2f\n" % (generated_seq_len / elapsed))  # :391-392
    out.flush()
    return None


def _emit(out, b):
    out.write(b.decode("utf-8", errors="replace") if isinstance(b, bytes) else b)
    out.flush()

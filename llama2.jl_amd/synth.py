"""Synthetic models of a given shape: seeded N(0, sigma) weights, norms = 1, quantized on the host
with the library's k-quant encoders.  Used by the tests and the benchmark (there are no
checkpoints to download); the reference has no counterpart (it cannot write models)."""
import os

import numpy as np

from . import _lib
from ._lib import TYPE_F32, TYPE_Q4_K, TYPE_Q5_K, TYPE_Q6_K
from .inference import LanguageModel, ModelConfig, TransformerLayerWeights, TransformerWeights
from .kquants import BLOCK_BYTES, QK_K, QuantMatrix
from .tokenizer import BPETokenizer

# tensor-type plans: role name -> ggml type
PLAN_F32 = dict.fromkeys(["emb", "output", "wq", "wk", "wv", "wo", "w1", "w2", "w3"], TYPE_F32)
PLAN_Q4_K_S = dict(PLAN_F32, **dict.fromkeys(["emb", "wq", "wk", "wv", "wo", "w1", "w2", "w3"], TYPE_Q4_K),
                   output=TYPE_Q6_K)
PLAN_Q5_K_M = dict(PLAN_F32, emb=TYPE_Q4_K, wq=TYPE_Q5_K, wk=TYPE_Q5_K, wv=TYPE_Q5_K, wo=TYPE_Q5_K, w1=TYPE_Q5_K,
                   w3=TYPE_Q5_K, w2=TYPE_Q6_K, output=TYPE_Q6_K)
PLAN_Q4_K = dict(PLAN_F32, **dict.fromkeys(["emb", "output", "wq", "wk", "wv", "wo", "w1", "w2", "w3"], TYPE_Q4_K))


def plan_q4_k_s_file(n_layers, n_first=None):
    """The tensor mix llama.cpp's quantizer is said to give a Q4_K_S file (not checked against a real file here):
    as PLAN_Q4_K_S, but attn_v and ffn_down of the first n_layers / 8 layers are q5_K.  A plan entry may be a
    list with one type per layer."""
    n_first = n_layers // 8 if n_first is None else n_first
    per_layer = [TYPE_Q5_K if l < n_first else TYPE_Q4_K for l in range(n_layers)]
    return dict(PLAN_Q4_K_S, wv=per_layer, w2=per_layer)


def plan_q4_k_m_file(n_layers):
    """The tensor mix llama.cpp's quantizer is said to give a Q4_K_M file (not checked against a real file here): q4_K
    layers in which attn_v and ffn_down are q6_K for the layers its "use more bits" rule picks (the first and the last
    eighth, and every third layer in between), q6_K output."""
    def more_bits(i):
        return i < n_layers // 8 or i >= 7 * n_layers // 8 or (i - n_layers // 8) % 3 == 2
    per_layer = [TYPE_Q6_K if more_bits(l) else TYPE_Q4_K for l in range(n_layers)]
    return dict(PLAN_Q4_K_S, wv=per_layer, w2=per_layer)


def _threads():
    return max(1, min(16, os.cpu_count() or 1))


def normal(seed, stream, shape, sigma=0.02, offset=0):
    n = int(np.prod(shape))
    out = np.empty(n, np.float32)
    rc = _lib.lib().l2h_synth_normal(seed, stream, offset, n, sigma, _lib.ptr(out), _threads())
    if rc != 0:
        raise _lib.L2HError(rc, "l2h_synth_normal failed")
    return out.reshape(shape)


def make_matrix(seed, stream, ne1, ne0, ggml_type, sigma=0.02, chunk_rows=None):
    """(ne1 out rows, ne0 in features) of N(0, sigma), as float32 or as a QuantMatrix.  Large
    matrices are generated and quantized in row chunks so that fp32 never exceeds ~1 GiB."""
    if ggml_type == TYPE_F32:
        return normal(seed, stream, (ne1, ne0), sigma)
    bb = BLOCK_BYTES[ggml_type]
    rb = (ne0 // QK_K) * bb
    out = np.empty(ne1 * rb, np.uint8)
    chunk_rows = chunk_rows or max(1, (1 << 28) // ne0)
    for r0 in range(0, ne1, chunk_rows):
        r1 = min(ne1, r0 + chunk_rows)
        x = normal(seed, stream, (r1 - r0, ne0), sigma, offset=r0 * ne0)
        rc = _lib.lib().l2h_quantize_weights(ggml_type, _lib.ptr(x), x.size, _lib.ptr(out[r0 * rb:r1 * rb]),
                                             _threads())
        if rc != 0:
            raise _lib.L2HError(rc, "l2h_quantize_weights failed")
    return QuantMatrix(ggml_type, out, ne0, ne1)


def dummy_tokenizer(vocab_size):
    """Byte-fallback style vocabulary: ids 0..2 are <unk>, <s>, </s>; then one token per id."""
    toks = [b"<unk>", b"<s>", b"</s>"] + [b" "] + [("<%d>" % i).encode() for i in range(4, vocab_size)]
    return BPETokenizer(toks[:vocab_size], [0.0] * vocab_size, 1, 2)


def synthetic_model(config, plan, seed=1234, sigma=0.02, share_classifier=False, norm_spread=0.2):
    """Random-init model of the given shape; stream ids are (layer, role) so any tensor can be
    regenerated alone.  The norm weights are seeded uniform(1 - norm_spread, 1 + norm_spread), different in
    every layer and tensor, so that a wrong layer's or the wrong tensor's norm weights change the result;
    norm_spread=0 gives all ones (what the benchmark configurations specify)."""
    c = config
    hs = c.dim // c.n_heads
    kv_dim = hs * c.n_kv_heads

    def mat(stream, ne1, ne0, role, layer=0):
        t = plan[role]
        return make_matrix(seed, stream, ne1, ne0, t[layer] if isinstance(t, (list, tuple)) else t, sigma)

    def norm(stream):
        if norm_spread == 0:
            return np.ones(c.dim, np.float32)
        rng = np.random.default_rng([seed, 7919, stream])
        return rng.uniform(1.0 - norm_spread, 1.0 + norm_spread, c.dim).astype(np.float32)

    emb = mat(1, c.vocab_size, c.dim, "emb")
    layers = []
    for l in range(c.n_layers):
        s = 100 + 16 * l
        layers.append(TransformerLayerWeights(
            rms_att_weight=norm(s + 7), rms_ffn_weight=norm(s + 8),
            wq=mat(s + 0, c.dim, c.dim, "wq", l), wk=mat(s + 1, kv_dim, c.dim, "wk", l), wv=mat(s + 2, kv_dim, c.dim, "wv", l),
            wo=mat(s + 3, c.dim, c.dim, "wo", l), w1=mat(s + 4, c.hidden_dim, c.dim, "w1", l),
            w2=mat(s + 5, c.dim, c.hidden_dim, "w2", l), w3=mat(s + 6, c.hidden_dim, c.dim, "w3", l)))
    output = emb if share_classifier else mat(2, c.vocab_size, c.dim, "output")
    weights = TransformerWeights(emb, layers, norm(3), output)
    return LanguageModel(c, dummy_tokenizer(c.vocab_size), weights)


def weight_bytes_per_token(model):
    """Bytes of weight data one decode step streams: every matvec tensor once (GGUF block bytes);
    norm weights and the embedding row are left out (<0.1 %)."""
    def nbytes(A):
        return A.data.size if isinstance(A, QuantMatrix) else A.size * 4
    w = model.weights
    total = nbytes(w.output_weight)
    for l in w.layers:
        total += sum(nbytes(getattr(l, n)) for n in ("wq", "wk", "wv", "wo", "w1", "w2", "w3"))
    return total


def seeded_prompt(seed, n, vocab_size):
    return np.random.default_rng(seed).integers(0, vocab_size, size=n).astype(np.int32)

"""llama2.c checkpoint / tokenizer.bin reader and writer (Llama2.jl src/load_karpathy.jl)."""
import struct

import numpy as np

from .inference import LanguageModel, ModelConfig, TransformerLayerWeights, TransformerWeights
from .tokenizer import BPETokenizer


def read_karpathy_config(f):
    """7 x Int32: dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len; rope base
    10000, interleaved RoPE (src/load_karpathy.jl:1-11)."""
    raw = f.read(28)
    if len(raw) != 28:
        raise ValueError("checkpoint too short for the 7-int header")
    dim, hidden, n_layers, n_heads, n_kv, vocab, seq = struct.unpack("<7i", raw)
    return ModelConfig(dim, hidden, n_layers, n_heads, n_kv, vocab, seq, 10000.0, False)


def read_karpathy_weights(f, c):
    """File order: emb, rms_att[L], wq[L], wk[L], wv[L], wo[L], rms_ffn[L], w1[L], w2[L], w3[L],
    rms_final (src/load_karpathy.jl:32-59).  Matrices on disk are (out, in) row-major.  As in the
    reference, wk and wv are read as (dim, dim) (:17-18), so only n_kv_heads == n_heads files load."""
    if c.n_kv_heads != c.n_heads:
        raise ValueError("llama2.c files with n_kv_heads != n_heads are not supported (wk/wv are read as dim x dim)")

    def arr(*shape):
        n = int(np.prod(shape))
        a = np.fromfile(f, dtype="<f4", count=n)
        if a.size != n:
            raise ValueError("checkpoint truncated")
        return a.reshape(shape)

    L = c.n_layers
    emb = arr(c.vocab_size, c.dim)
    rms_att = arr(L, c.dim)
    wq, wk, wv, wo = arr(L, c.dim, c.dim), arr(L, c.dim, c.dim), arr(L, c.dim, c.dim), arr(L, c.dim, c.dim)
    rms_ffn = arr(L, c.dim)
    w1, w2, w3 = arr(L, c.hidden_dim, c.dim), arr(L, c.dim, c.hidden_dim), arr(L, c.hidden_dim, c.dim)
    rms_final = arr(c.dim)
    layers = [TransformerLayerWeights(rms_att[l], rms_ffn[l], wq[l], wk[l], wv[l], wo[l], w1[l], w2[l], w3[l])
              for l in range(L)]
    # the classifier shares the embedding (:56)
    return TransformerWeights(emb, layers, rms_final, emb)


def load_karpathy_tokenizer(filename, vocab_size):
    """Int32 max_token_length, then per token Float32 score, Int32 len, bytes
    (src/load_karpathy.jl:61-78); bos = 1, eos = 2 (0-based; the reference's 2 and 3)."""
    tokens, scores = [], []
    with open(filename, "rb") as f:
        f.read(4)
        for _ in range(vocab_size):
            score, n = struct.unpack("<fi", f.read(8))
            tokens.append(f.read(n))
            scores.append(score)
    return BPETokenizer(tokens, scores, 1, 2)


def load_karpathy_model(checkpoint_filename, tokenizer_filename):
    """load_karpathy_model(checkpoint, tokenizer) (src/load_karpathy.jl:80-98)."""
    with open(checkpoint_filename, "rb") as f:
        config = read_karpathy_config(f)
        weights = read_karpathy_weights(f, config)
    tokenizer = load_karpathy_tokenizer(tokenizer_filename, config.vocab_size)
    return LanguageModel(config, tokenizer, weights)


def save_karpathy_model(checkpoint_filename, tokenizer_filename, model):
    c, w = model.config, model.weights
    with open(checkpoint_filename, "wb") as f:
        f.write(struct.pack("<7i", c.dim, c.hidden_dim, c.n_layers, c.n_heads, c.n_kv_heads, c.vocab_size, c.seq_len))

        def put(a):
            np.ascontiguousarray(a, dtype="<f4").tofile(f)

        put(w.token_embedding_table)
        for name in ("rms_att_weight", "wq", "wk", "wv", "wo", "rms_ffn_weight", "w1", "w2", "w3"):
            for l in w.layers:
                put(getattr(l, name))
        put(w.rms_final_weight)
    tok = model.tokenizer
    with open(tokenizer_filename, "wb") as f:
        f.write(struct.pack("<i", max(len(t) for t in tok.id_to_token)))
        for t, s in zip(tok.id_to_token, tok.token_scores):
            f.write(struct.pack("<fi", s, len(t)) + t)

"""GGUF reader/writer for the subset Llama2.jl loads (src/load_gguf.jl).

load_gguf_model(filename; mmap=true) keeps the reference's behaviour: metadata value types
STRING/UINT32/INT32/FLOAT32/BOOL/ARRAY only (:59-77), tensor types F32/Q4_K/Q5_K/Q6_K only
(:135-185), architectures "llama" and "phi3" (:383-391), tokenizer models "llama" and "gpt2"
(:345-371).  One extension: `seq_len` (the reference hard-codes 512, :237,:299).
"""
import struct

import numpy as np

from .inference import LanguageModel, ModelConfig, TransformerLayerWeights, TransformerWeights
from .kquants import BLOCK_BYTES, QK_K, QuantMatrix
from .tokenizer import BPETokenizer

# GGUF_METADATA_VALUE_TYPE (src/load_gguf.jl:1-24)
(T_UINT8, T_INT8, T_UINT16, T_INT16, T_UINT32, T_INT32, T_FLOAT32, T_BOOL, T_STRING, T_ARRAY, T_UINT64, T_INT64,
 T_FLOAT64) = range(13)
# GGML_TYPE (:26-42)
GGML_F32, GGML_F16, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K = 0, 1, 12, 13, 14
# LLAMA_TOKEN_TYPE (:44-52)
TOKEN_NORMAL, TOKEN_BYTE = 1, 6


class GGUFError(ValueError):
    pass


class _Reader:
    def __init__(self, buf):
        self.buf, self.pos = buf, 0

    def take(self, fmt):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise GGUFError("unexpected end of file")
        v = struct.unpack_from(fmt, self.buf, self.pos)[0]
        self.pos += size
        return v

    def string(self):  # read_gguf_string, :54-57
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise GGUFError("unexpected end of file")
        b = bytes(self.buf[self.pos:self.pos + n])
        self.pos += n
        return b

    def value(self, vt):  # read_gguf_metadata_value, :59-77
        if vt == T_STRING:
            return self.string()
        if vt == T_UINT32:
            return self.take("<I")
        if vt == T_INT32:
            return self.take("<i")
        if vt == T_FLOAT32:
            return self.take("<f")
        if vt == T_ARRAY:
            at = self.take("<I")
            n = self.take("<Q")
            return [self.value(at) for _ in range(n)]
        if vt == T_BOOL:
            return self.take("<?")
        raise GGUFError("reading metadata value of type %d is not implemented yet" % vt)


def align_offset(offset, alignment):  # :131-133
    return offset + (alignment - (offset % alignment)) % alignment


def read_gguf(filename, mmap=True):
    """Returns (metadata dict, {name: tensor}); k-quant tensors are QuantMatrix, F32 tensors are
    float32 arrays of shape reversed(dims) (so a matrix is (out, in))."""
    raw = np.memmap(filename, dtype=np.uint8, mode="r") if mmap else np.fromfile(filename, dtype=np.uint8)
    r = _Reader(raw)
    if bytes(raw[:4]) != b"GGUF":
        raise GGUFError("Not a GGUF file")  # :87-89
    r.pos = 4
    r.take("<I")  # version: read, never checked (:91)
    tensor_count = r.take("<Q")
    kv_count = r.take("<Q")
    meta = {}
    for _ in range(kv_count):  # :96-102
        key = r.string().decode("utf-8")
        vt = r.take("<I")
        meta[key] = r.value(vt)
    infos = []
    for _ in range(tensor_count):  # read_gguf_tensor_info, :121-129
        name = r.string().decode("utf-8")
        nd = r.take("<I")
        dims = [r.take("<Q") for _ in range(nd)]
        typ = r.take("<I")
        off = r.take("<Q")
        infos.append((name, dims, typ, off))
    alignment = meta.get("general.alignment", 32)  # :327
    base = align_offset(r.pos, alignment)  # :328
    tensors = {}
    for name, dims, typ, off in infos:  # :331-334
        start = base + off
        n = 1
        for d in dims:
            n *= d
        if typ == GGML_F32:
            nbytes = 4 * n
            if start + nbytes > raw.size:
                raise GGUFError("tensor %s runs past the end of the file" % name)
            arr = raw[start:start + nbytes].view(np.float32).reshape(tuple(reversed(dims)))
            tensors[name] = arr if mmap else np.array(arr)
        elif typ in (GGML_Q4_K, GGML_Q5_K, GGML_Q6_K):
            if dims[0] % QK_K != 0:
                raise GGUFError("tensor %s: ne0 = %d is not a multiple of %d" % (name, dims[0], QK_K))  # :141
            ne1 = n // dims[0]
            nbytes = (n // QK_K) * BLOCK_BYTES[typ]
            if start + nbytes > raw.size:
                raise GGUFError("tensor %s runs past the end of the file" % name)
            tensors[name] = QuantMatrix(typ, raw[start:start + nbytes], dims[0], ne1)
        else:
            raise GGUFError("tensor type %d not implemented" % typ)  # :153,:179
    return meta, tensors


def gpt2_decoder():
    """Inverse of GPT-2's byte-to-unicode table (src/load_gguf.jl:195-209)."""
    bs = list(range(ord("!"), ord("~") + 1)) + list(range(0xA1, 0xAC + 1)) + list(range(0xAE, 0xFF + 1))
    cs = bs[:]
    n = 0
    for b in range(256):
        if b not in bs:
            bs.append(b)
            cs.append(256 + n)
            n += 1
    return {chr(c): b for c, b in zip(cs, bs)}


def _layer(tensors, i, arch):
    p = "blk.%d." % i
    if arch == "llama":  # build_llama_weights_layer, :211-227
        if p + "attn_q.weight" not in tensors:
            raise GGUFError("missing blk.%d weights" % i)
        return TransformerLayerWeights(
            rms_att_weight=tensors[p + "attn_norm.weight"], rms_ffn_weight=tensors[p + "ffn_norm.weight"],
            wq=tensors[p + "attn_q.weight"], wk=tensors[p + "attn_k.weight"], wv=tensors[p + "attn_v.weight"],
            wo=tensors[p + "attn_output.weight"], w1=tensors[p + "ffn_gate.weight"],
            w2=tensors[p + "ffn_down.weight"], w3=tensors[p + "ffn_up.weight"])
    # phi3: fused qkv and gate+up, split along the output rows (build_phi3_weights_layer, :255-289)
    if p + "attn_qkv.weight" not in tensors:
        raise GGUFError("missing blk.%d weights" % i)
    wqkv = tensors[p + "attn_qkv.weight"]
    n = _rows(wqkv) // 3
    gu = tensors[p + "ffn_up.weight"]
    h = _rows(gu) // 2
    return TransformerLayerWeights(
        rms_att_weight=tensors[p + "attn_norm.weight"], rms_ffn_weight=tensors[p + "ffn_norm.weight"],
        wq=_row_range(wqkv, 0, n), wk=_row_range(wqkv, n, 2 * n), wv=_row_range(wqkv, 2 * n, 3 * n),
        wo=tensors[p + "attn_output.weight"], w1=_row_range(gu, 0, h), w2=tensors[p + "ffn_down.weight"],
        w3=_row_range(gu, h, 2 * h))


def _rows(t):
    return t.ne1 if isinstance(t, QuantMatrix) else t.shape[0]


def _row_range(t, a, b):
    return t.rows(a, b) if isinstance(t, QuantMatrix) else t[a:b]


def load_gguf_model(filename, mmap=True, seq_len=512):
    """load_gguf_model(filename; mmap=true) (src/load_gguf.jl:317-394)."""
    meta, tensors = read_gguf(filename, mmap)
    id_to_token = list(meta["tokenizer.ggml.tokens"])  # :340
    token_types = meta["tokenizer.ggml.token_type"]
    tok_model = meta["tokenizer.ggml.model"]
    if tok_model == b"llama":  # :345-358
        for i, t in enumerate(id_to_token):
            if token_types[i] == TOKEN_NORMAL:
                id_to_token[i] = t.replace(b"\xe2\x96\x81", b" ")
            elif token_types[i] == TOKEN_BYTE:
                id_to_token[i] = bytes([int(t[1:-1].decode(), 0)])  # "<0xNN>"
    elif tok_model == b"gpt2":  # :359-368
        dec = gpt2_decoder()
        for i, t in enumerate(id_to_token):
            if token_types[i] == TOKEN_NORMAL:
                id_to_token[i] = bytes(dec[ch] for ch in t.decode("utf-8"))
    else:
        raise GGUFError("unsupported tokenizer model: %s" % tok_model.decode(errors="replace"))
    tokenizer = BPETokenizer(id_to_token, meta["tokenizer.ggml.scores"], meta["tokenizer.ggml.bos_token_id"],
                             meta["tokenizer.ggml.eos_token_id"])  # :373-380 (ids stay 0-based here)
    vocab_size = len(id_to_token)
    arch = meta["general.architecture"].decode()
    if arch not in ("llama", "phi3"):
        raise GGUFError("unsupported model architecture: %s" % arch)  # :389
    config = ModelConfig(  # build_llama :229-240, build_phi3 :291-302
        dim=meta[arch + ".embedding_length"], hidden_dim=meta[arch + ".feed_forward_length"],
        n_layers=meta[arch + ".block_count"], n_heads=meta[arch + ".attention.head_count"],
        n_kv_heads=meta[arch + ".attention.head_count_kv"], vocab_size=vocab_size, seq_len=seq_len,
        rope_freq_base=meta.get(arch + ".rope.freq_base", 10000.0), rope_is_neox=(arch == "phi3"))
    layers = [_layer(tensors, i, arch) for i in range(config.n_layers)]
    weights = TransformerWeights(token_embedding_table=tensors["token_embd.weight"], layers=layers,
                                 rms_final_weight=tensors["output_norm.weight"],
                                 output_weight=tensors["output.weight"])  # no tied-embedding fallback (:248)
    return LanguageModel(config, tokenizer, weights)


# ------------------------------------------------------------------------------------------------
# writer (for synthetic models; stays inside the subset the reader above accepts)
# ------------------------------------------------------------------------------------------------
def _w_string(b):
    b = b if isinstance(b, bytes) else b.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _w_value(v, vt=None):
    if vt is None:
        if isinstance(v, bool):
            vt = T_BOOL
        elif isinstance(v, (bytes, str)):
            vt = T_STRING
        elif isinstance(v, float):
            vt = T_FLOAT32
        elif isinstance(v, int):
            vt = T_UINT32
        elif isinstance(v, (list, tuple)):
            vt = T_ARRAY
        else:
            raise TypeError(type(v))
    if vt == T_STRING:
        return vt, _w_string(v)
    if vt == T_UINT32:
        return vt, struct.pack("<I", v)
    if vt == T_INT32:
        return vt, struct.pack("<i", v)
    if vt == T_FLOAT32:
        return vt, struct.pack("<f", v)
    if vt == T_BOOL:
        return vt, struct.pack("<?", v)
    if vt == T_ARRAY:
        if len(v) == 0:
            return vt, struct.pack("<IQ", T_UINT32, 0)
        et, _ = _w_value(v[0])
        return vt, struct.pack("<IQ", et, len(v)) + b"".join(_w_value(e, et)[1] for e in v)
    raise TypeError("metadata value type %d is outside the readable subset" % vt)


def write_gguf(filename, meta, tensors, alignment=32, typed_meta=None):
    """meta: {key: value}; typed_meta: {key: (type, value)} for explicit types (e.g. INT32).
    tensors: list of (name, tensor) with tensor a QuantMatrix or float32 array ((out, in) or 1-D)."""
    head = b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(meta) + len(typed_meta or {}))
    for k, v in meta.items():
        vt, payload = _w_value(v)
        head += _w_string(k) + struct.pack("<I", vt) + payload
    for k, (vt, v) in (typed_meta or {}).items():
        _, payload = _w_value(v, vt)
        head += _w_string(k) + struct.pack("<I", vt) + payload
    infos, off, blobs = b"", 0, []
    for name, t in tensors:
        if isinstance(t, QuantMatrix):
            dims, typ, data = [t.ne0, t.ne1], t.type, np.ascontiguousarray(t.data)
        else:
            a = np.ascontiguousarray(t, dtype=np.float32)
            dims, typ, data = list(reversed(a.shape)), GGML_F32, a.reshape(-1).view(np.uint8)
        infos += _w_string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        infos += struct.pack("<IQ", typ, off)
        blobs.append((off, data))
        off = align_offset(off + data.size, alignment)
    with open(filename, "wb") as f:
        f.write(head + infos)
        base = align_offset(f.tell(), alignment)
        f.write(b"\0" * (base - f.tell()))
        for o, data in blobs:
            f.write(b"\0" * (base + o - f.tell()))
            data.tofile(f)


def save_gguf_model(filename, model, arch="llama", tokens=None, fused_phi3=True):
    """Writes a LanguageModel as a GGUF file the loader above (and the reference's) reads back."""
    c, w = model.config, model.weights
    tok = model.tokenizer
    if tokens is None:
        tokens = [bytes(t) for t in tok.id_to_token]
    meta = {
        "general.architecture": arch,
        arch + ".embedding_length": c.dim, arch + ".feed_forward_length": c.hidden_dim,
        arch + ".block_count": c.n_layers, arch + ".attention.head_count": c.n_heads,
        arch + ".attention.head_count_kv": c.n_kv_heads, arch + ".rope.freq_base": float(c.rope_freq_base),
        "tokenizer.ggml.model": "llama", "tokenizer.ggml.tokens": tokens,
        "tokenizer.ggml.scores": [float(s) for s in tok.token_scores],
        "tokenizer.ggml.bos_token_id": tok.bos_token_id, "tokenizer.ggml.eos_token_id": tok.eos_token_id,
    }
    typed = {"tokenizer.ggml.token_type": (T_ARRAY, [0] * len(tokens))}
    ts = [("token_embd.weight", w.token_embedding_table), ("output_norm.weight", w.rms_final_weight),
          ("output.weight", w.output_weight)]
    for i, l in enumerate(w.layers):
        p = "blk.%d." % i
        ts += [(p + "attn_norm.weight", l.rms_att_weight), (p + "ffn_norm.weight", l.rms_ffn_weight)]
        if arch == "phi3" and fused_phi3:
            ts += [(p + "attn_qkv.weight", _concat_rows([l.wq, l.wk, l.wv])),
                   (p + "ffn_up.weight", _concat_rows([l.w1, l.w3]))]
        else:
            ts += [(p + "attn_q.weight", l.wq), (p + "attn_k.weight", l.wk), (p + "attn_v.weight", l.wv),
                   (p + "ffn_gate.weight", l.w1), (p + "ffn_up.weight", l.w3)]
        ts += [(p + "attn_output.weight", l.wo), (p + "ffn_down.weight", l.w2)]
    write_gguf(filename, meta, ts, typed_meta=typed)


def _concat_rows(ms):
    if isinstance(ms[0], QuantMatrix):
        return QuantMatrix(ms[0].type, np.concatenate([m.data for m in ms]), ms[0].ne0, sum(m.ne1 for m in ms))
    return np.concatenate(ms, axis=0)

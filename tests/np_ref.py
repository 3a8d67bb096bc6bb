"""Independent numpy restatement of the reference's codecs and operators, written from the text of
Llama2.jl (src/kquants.jl, src/inference.jl) without looking at oracle/l2c.c's structure: vectorised
over blocks, float64 where the reference's summation order is free.  Used to pin the C oracle
(two restatements of the same text must agree) and to make the golden vectors in tests/golden/.
"""
import numpy as np

QK_K = 256

q4_dtype = np.dtype([("d", "<f2"), ("dmin", "<f2"), ("scales", "u1", 12), ("qs", "u1", 128)])
q5_dtype = np.dtype([("d", "<f2"), ("dmin", "<f2"), ("scales", "u1", 12), ("qh", "u1", 32), ("qs", "u1", 128)])
q6_dtype = np.dtype([("ql", "u1", 128), ("qh", "u1", 64), ("scales", "i1", 16), ("d", "<f2")])
q8_dtype = np.dtype([("d", "<f4"), ("qs", "i1", 256), ("bsums", "<i2", 16)])


def scales_k4(sc12):
    """(n,12) uint8 -> (sc, m) each (n,8): kquants.jl:80-81,86-87 (sub-blocks 1..4, one-based) and
    :102-103,108-109 (5..8)."""
    s = sc12.astype(np.int32)
    sc = np.zeros(s.shape[:-1] + (8,), np.int32)
    m = np.zeros_like(sc)
    for j in range(1, 9):  # one-based like the Julia text
        if j <= 4:
            sc[..., j - 1] = s[..., j - 1] & 63
            m[..., j - 1] = s[..., j - 1 + 4] & 63
        else:
            sc[..., j - 1] = (s[..., j - 1 + 4] & 0xF) | ((s[..., j - 1 - 4] >> 6) << 4)
            m[..., j - 1] = (s[..., j - 1 + 4] >> 4) | ((s[..., j - 1] >> 6) << 4)
    return sc, m


def ints_q4(blocks):
    """(n,) blocks -> unsigned quants (n,256) in element order (kquants.jl:92-98)."""
    qs = blocks["qs"].astype(np.int32).reshape(-1, 4, 32)
    q = np.empty((qs.shape[0], 4, 64), np.int32)
    q[:, :, :32] = qs & 0xF
    q[:, :, 32:] = qs >> 4
    return q.reshape(-1, 256)


def ints_q5(blocks):
    q = ints_q4(blocks).reshape(-1, 8, 32)
    qh = blocks["qh"].astype(np.int32)  # (n,32); bit s of qh[l] belongs to sub-block s (kquants.jl:196-221)
    for s in range(8):
        q[:, s, :] += np.where((qh >> s) & 1, 16, 0)
    return q.reshape(-1, 256)


def ints_q6(blocks):
    """signed quants q-32 (n,256) (kquants.jl:333-336)."""
    ql = blocks["ql"].astype(np.int32).reshape(-1, 2, 64)
    qh = blocks["qh"].astype(np.int32).reshape(-1, 2, 32)
    q = np.empty((ql.shape[0], 2, 4, 32), np.int32)
    q[:, :, 0] = (ql[:, :, :32] & 0xF) | (((qh >> 0) & 3) << 4)
    q[:, :, 1] = (ql[:, :, 32:] & 0xF) | (((qh >> 2) & 3) << 4)
    q[:, :, 2] = (ql[:, :, :32] >> 4) | (((qh >> 4) & 3) << 4)
    q[:, :, 3] = (ql[:, :, 32:] >> 4) | (((qh >> 6) & 3) << 4)
    return q.reshape(-1, 256) - 32


def dequant_q45(blocks, q):
    d = blocks["d"].astype(np.float32)[:, None]
    dmin = blocks["dmin"].astype(np.float32)[:, None]
    sc, m = scales_k4(blocks["scales"])
    d1 = (d * sc.astype(np.float32)).astype(np.float32)  # kquants.jl:83
    m1 = (dmin * m.astype(np.float32)).astype(np.float32)  # :84
    q = q.reshape(-1, 8, 32).astype(np.float32)
    y = (d1[:, :, None] * q).astype(np.float32) - m1[:, :, None]  # :93
    return y.astype(np.float32).reshape(-1)


def dequant_q4(raw):
    b = np.frombuffer(np.ascontiguousarray(raw), q4_dtype)
    return dequant_q45(b, ints_q4(b))


def dequant_q5(raw):
    b = np.frombuffer(np.ascontiguousarray(raw), q5_dtype)
    return dequant_q45(b, ints_q5(b))


def q6_scale_index():
    """element e (0..255) -> index of its int8 scale: 8n + l//16 + 2g (kquants.jl:338-343,352-357)."""
    e = np.arange(256)
    n, r = e // 128, e % 128
    g, l = r // 32, r % 32
    return 8 * n + l // 16 + 2 * g


def dequant_q6(raw):
    b = np.frombuffer(np.ascontiguousarray(raw), q6_dtype)
    q = ints_q6(b)
    sc = b["scales"].astype(np.int32)[:, q6_scale_index()]
    d = b["d"].astype(np.float32)[:, None]
    return (d * (sc * q).astype(np.float32)).astype(np.float32).reshape(-1)  # :340


DEQUANT = {12: dequant_q4, 13: dequant_q5, 14: dequant_q6}


def quantize_q8(x):
    """llama.cpp quantize_row_q8_K_ref: first element of largest magnitude, iscale = -127/max,
    round-half-even, min(127, .), bsums, d = 1/iscale."""
    x = np.asarray(x, np.float32).reshape(-1, 256)
    out = np.zeros(x.shape[0], q8_dtype)
    for i, blk in enumerate(x):
        ax = np.abs(blk)
        j = int(np.argmax(ax))  # first maximum
        if ax[j] == 0:
            continue
        iscale = np.float32(-127.0) / blk[j]
        q = np.minimum(127, np.rint((iscale * blk).astype(np.float32))).astype(np.int32)
        out[i]["qs"] = q.astype(np.int8)
        out[i]["bsums"] = q.reshape(16, 16).sum(1).astype(np.int16)
        out[i]["d"] = np.float32(1.0) / iscale
    return out


def block_ints(typ, raw, q8):
    """per-block (I_sc, I_min) by brute force on the integer fields."""
    if typ == 14:
        b = np.frombuffer(np.ascontiguousarray(raw), q6_dtype)
        q = ints_q6(b).astype(np.int64)
        sc = b["scales"].astype(np.int64)[:, q6_scale_index()]
        return (sc * q * q8["qs"].astype(np.int64)).sum(1), np.zeros(len(b), np.int64)
    b = np.frombuffer(np.ascontiguousarray(raw), q4_dtype if typ == 12 else q5_dtype)
    q = (ints_q4(b) if typ == 12 else ints_q5(b)).astype(np.int64).reshape(-1, 8, 32)
    sc, m = scales_k4(b["scales"])
    x = q8["qs"].astype(np.int64).reshape(-1, 8, 32)
    i_sc = (sc.astype(np.int64) * (q * x).sum(2)).sum(1)
    bs = q8["bsums"].astype(np.int64).reshape(-1, 8, 2).sum(2)
    return i_sc, (m.astype(np.int64) * bs).sum(1)


def vecdot_q8(typ, raw, q8):
    """row value in exact arithmetic (python floats = fp64 on fp32-rounded factors), fp32 at the end"""
    dt = {12: q4_dtype, 13: q5_dtype, 14: q6_dtype}[typ]
    b = np.frombuffer(np.ascontiguousarray(raw), dt)
    i_sc, i_min = block_ints(typ, raw, q8)
    d = b["d"].astype(np.float32)
    dy = (d * q8["d"]).astype(np.float32).astype(np.float64)
    s = (dy * i_sc).sum()
    if typ != 14:
        my = (b["dmin"].astype(np.float32) * q8["d"]).astype(np.float32).astype(np.float64)
        s -= (my * i_min).sum()
    return np.float32(s)


# ---- operators (float64 closed forms; src/inference.jl:102-220,295-299) --------------------------
def rmsnorm(x, w):
    x = np.asarray(x, np.float64)
    return np.asarray(w, np.float64) * (x / np.sqrt(np.mean(x * x) + 1e-5))


def rope(x, hs, pos0, base, neox):
    x = np.asarray(x, np.float64).reshape(-1, hs).copy()
    half = hs // 2
    theta = pos0 * (float(base) ** (-np.arange(half) / half))
    c, s = np.cos(theta), np.sin(theta)
    if neox:
        a, b = x[:, :half].copy(), x[:, half:].copy()
        x[:, :half], x[:, half:] = a * c - b * s, a * s + b * c
    else:
        a, b = x[:, 0::2].copy(), x[:, 1::2].copy()
        x[:, 0::2], x[:, 1::2] = a * c - b * s, a * s + b * c
    return x.reshape(-1)


def softmax(x):
    x = np.asarray(x, np.float64)
    e = np.exp(x - x.max())
    return e / e.sum()


def attention(q, kc, vc, hs, n_heads, n_kv):
    q = np.asarray(q, np.float64).reshape(n_heads, hs)
    kc = np.asarray(kc, np.float64).reshape(-1, n_kv, hs)
    vc = np.asarray(vc, np.float64).reshape(-1, n_kv, hs)
    out = np.zeros((n_heads, hs))
    g = n_heads // n_kv
    for h in range(n_heads):
        a = softmax(kc[:, h // g, :] @ q[h] / np.sqrt(hs))
        out[h] = a @ vc[:, h // g, :]
    return out.reshape(-1)


def swiglu(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return a / (1 + np.exp(-a)) * b


def transformer_f32(cfg, W, tokens):
    """float64 forward of an F32 model over a token sequence; returns the logits of every position.
    W: dict with emb, rms_final, output, and per-layer lists (src/inference.jl:222-315)."""
    dim, hs = cfg["dim"], cfg["dim"] // cfg["n_heads"]
    n_kv, n_heads = cfg["n_kv_heads"], cfg["n_heads"]
    kv_dim = hs * n_kv
    L = cfg["n_layers"]
    kc = [np.zeros((0, kv_dim)) for _ in range(L)]
    vc = [np.zeros((0, kv_dim)) for _ in range(L)]
    outs = []
    f = lambda a: np.asarray(a, np.float64)
    for pos, tok in enumerate(tokens):
        x = f(W["emb"][tok]).copy()
        for l in range(L):
            xb = rmsnorm(x, W["rms_att"][l])
            q, k, v = f(W["wq"][l]) @ xb, f(W["wk"][l]) @ xb, f(W["wv"][l]) @ xb
            q = rope(q, hs, pos, cfg["rope_freq_base"], cfg["rope_is_neox"])
            k = rope(k, hs, pos, cfg["rope_freq_base"], cfg["rope_is_neox"])
            kc[l] = np.vstack([kc[l], k[None]])
            vc[l] = np.vstack([vc[l], v[None]])
            att = attention(q, kc[l], vc[l], hs, n_heads, n_kv)
            x = x + f(W["wo"][l]) @ att
            xb = rmsnorm(x, W["rms_ffn"][l])
            hb = swiglu(f(W["w1"][l]) @ xb, f(W["w3"][l]) @ xb)
            x = x + f(W["w2"][l]) @ hb
        x = rmsnorm(x, W["rms_final"])
        outs.append(f(W["output"]) @ x)
    return np.array(outs)

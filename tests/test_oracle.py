"""Pins the CPU oracle (oracle/l2c.c).  The reference ships no tests or vectors, so the oracle is
checked against (1) hand-built blocks with closed-form expected values (tests/golden), (2) an
independent numpy restatement written from the same Julia text (tests/np_ref.py), (3) identities
the reference implies (vecdot == dot(dequantize)), (4) float64 closed forms of every operator and
of the whole transformer, (5) closed-form properties of the q8_K quantizer and brute force for
the integer dot products.  No GPU needed.
"""
import json
import os

import numpy as np
import pytest

import np_ref

HERE = os.path.dirname(os.path.abspath(__file__))
Q4, Q5, Q6, F32 = 12, 13, 14, 0
BB = {Q4: 144, Q5: 176, Q6: 210}


def rand_blocks(rng, typ, n):
    raw = rng.integers(0, 256, size=(n, BB[typ]), dtype=np.uint8)
    d = rng.uniform(-0.02, 0.02, size=(n, 2)).astype(np.float16).view(np.uint8)
    if typ == Q6:
        raw[:, 208:210] = d[:, :2]
    else:
        raw[:, 0:4] = d
    return raw.reshape(-1)


def rel(a, b):
    return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64))) / max(1e-30, np.max(np.abs(b))))


def test_block_sizes(orc):
    # src/kquants.jl:7-42
    assert [orc.lib().l2c_block_bytes(t) for t in (F32, Q4, Q5, Q6)] == [4, 144, 176, 210]
    assert orc.block_q8_K.itemsize == 292 and np_ref.q8_dtype.itemsize == 292
    assert np_ref.q4_dtype.itemsize == 144 and np_ref.q5_dtype.itemsize == 176 and np_ref.q6_dtype.itemsize == 210


def test_golden_vectors(orc):
    vecs = json.load(open(os.path.join(HERE, "golden", "kquant_vectors.json")))
    assert len(vecs) >= 7
    for v in vecs:
        raw = np.frombuffer(bytes.fromhex(v["raw"]), np.uint8)
        want = np.array(v["expected"], np.float32)
        got = orc.dequantize(v["type"], raw)
        assert np.array_equal(got, want), v["name"]
        assert np.array_equal(np_ref.DEQUANT[v["type"]](raw), want), v["name"] + " (numpy restatement)"


def test_fp16_conversion_exhaustive(orc):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([orc.lib().l2c_fp16_to_fp32(int(x)) for x in h], np.float32)
    ok = np.isnan(want) | (got.view(np.uint32) == want.view(np.uint32))
    assert ok.all()


def test_scale_unpack_every_bit(orc, rng):
    """Toggle each of the 96 bits of the packed scales alone: exactly one 6-bit field changes."""
    import ctypes
    base = np.zeros(12, np.uint8)
    sc, m = np.zeros(8, np.uint8), np.zeros(8, np.uint8)
    for bit in range(96):
        p = base.copy()
        p[bit // 8] = 1 << (bit % 8)
        orc.lib().l2c_scale_min_k4(p.ctypes.data_as(ctypes.c_void_p), sc.ctypes.data_as(ctypes.c_void_p),
                                   m.ctypes.data_as(ctypes.c_void_p))
        rsc, rm = np_ref.scales_k4(p[None])
        assert np.array_equal(sc, rsc[0]) and np.array_equal(m, rm[0])
        assert np.count_nonzero(sc) + np.count_nonzero(m) == 1
    for _ in range(200):
        p = rng.integers(0, 256, 12, dtype=np.uint8)
        orc.lib().l2c_scale_min_k4(p.ctypes.data_as(ctypes.c_void_p), sc.ctypes.data_as(ctypes.c_void_p),
                                   m.ctypes.data_as(ctypes.c_void_p))
        rsc, rm = np_ref.scales_k4(p[None])
        assert np.array_equal(sc, rsc[0]) and np.array_equal(m, rm[0]) and sc.max() < 64 and m.max() < 64


@pytest.mark.parametrize("typ", [Q4, Q5, Q6])
def test_dequantize_matches_numpy_restatement(orc, rng, typ):
    raw = rand_blocks(rng, typ, 4000)
    assert np.array_equal(orc.dequantize(typ, raw).view(np.uint32), np_ref.DEQUANT[typ](raw).view(np.uint32))


@pytest.mark.parametrize("typ", [Q4, Q5, Q6])
def test_vecdot_is_dot_of_dequantized(orc, rng, typ):
    """The reference states the weight expression twice, in dequantize! and in vecdot
    (src/kquants.jl:93 vs :152 etc.): vecdot(x, y) == dot(dequantize(x), y)."""
    nb = 16
    raw = rand_blocks(rng, typ, nb)
    y = rng.standard_normal(nb * 256).astype(np.float32)
    w = orc.dequantize(typ, raw)
    exact = float(np.dot(w.astype(np.float64), y.astype(np.float64)))
    assert orc.vecdot_f32act(typ, raw, y, canon=1) == np.float32(exact)
    seq = np.float32(0)
    for a, b in zip(w, y):
        seq = np.float32(seq + np.float32(b * a))
    assert orc.vecdot_f32act(typ, raw, y, canon=0) == seq
    assert abs(orc.vecdot_f32act(typ, raw, y, canon=0) - exact) <= 1e-4 * np.abs(w * y).sum()


def test_q8k_properties(orc, rng):
    x = (rng.standard_normal(256 * 50) * rng.uniform(0.01, 100, 50).repeat(256)).astype(np.float32)
    x[256 * 3:256 * 4] = 0
    i, j = 256 * 5 + 7, 256 * 5 + 100  # tie of the extreme inside block 5: the first (negative) one fixes the sign
    x[256 * 5:256 * 6] = rng.uniform(-1, 1, 256)
    x[i], x[j] = -3.0, 3.0
    q = orc.quantize_q8_K(x)
    assert q.tobytes() == np_ref.quantize_q8(x).tobytes()
    for b in range(50):
        blk = x[256 * b:256 * b + 256]
        if not blk.any():
            assert q[b]["d"] == 0 and not q[b]["qs"].any() and not q[b]["bsums"].any()
            continue
        k = int(np.argmax(np.abs(blk)))
        assert q[b]["qs"][k] == -127  # iscale = -127/max maps the extreme to -127
        assert np.all(np.abs(q[b]["qs"].astype(np.float64) * q[b]["d"] - blk) <= abs(q[b]["d"]) * 0.5000001)
        assert np.array_equal(q[b]["bsums"], q[b]["qs"].astype(np.int32).reshape(16, 16).sum(1))
        assert np.sign(q[b]["d"]) == -np.sign(blk[k])
    assert q[5]["qs"][7] == -127 and q[5]["qs"][100] == 127 and q[5]["d"] > 0


@pytest.mark.parametrize("typ", [Q4, Q5, Q6])
def test_integer_dots_brute_force(orc, rng, typ):
    nb = 24
    raw = rand_blocks(rng, typ, nb)
    x = rng.standard_normal(nb * 256).astype(np.float32)
    q8 = orc.quantize_q8_K(x)
    v, isc, imin = orc.vecdot_q8k(typ, raw, q8, canon=1)
    w_isc, w_imin = np_ref.block_ints(typ, raw, q8)
    assert np.array_equal(isc, w_isc) and np.array_equal(imin, w_imin)
    assert np.float32(v) == np_ref.vecdot_q8(typ, raw, q8)
    # the q8_K path approximates the float path to the quantization step of the activations
    f = orc.vecdot_f32act(typ, raw, x, canon=1)
    w = orc.dequantize(typ, raw)
    assert abs(v - f) <= 0.02 * np.sqrt((w.astype(np.float64) ** 2).sum()) * np.abs(x).max() / 127 * 16


def test_matmul_rows_and_threads(orc, rng):
    ne0, ne1 = 512, 37
    raw = rand_blocks(rng, Q4, ne1 * 2)
    x = rng.standard_normal(ne0).astype(np.float32)
    for mode in (0, 1, 2, 3):
        y1 = orc.matmul(Q4, raw, ne0, ne1, x, mode, nthreads=1)
        y8 = orc.matmul(Q4, raw, ne0, ne1, x, mode, nthreads=8)
        assert np.array_equal(y1.view(np.uint32), y8.view(np.uint32))  # rows are independent (src/matmul.jl:18)
    rb = 2 * 144
    for i in (0, 17, 36):
        assert orc.matmul(Q4, raw, ne0, ne1, x, 0)[i] == np.float32(orc.vecdot_f32act(Q4, raw[i * rb:(i + 1) * rb], x, 0))
    A = rng.standard_normal((ne1, ne0)).astype(np.float32)
    assert rel(orc.matmul(F32, A, ne0, ne1, x, 0), A.astype(np.float64) @ x) < 1e-5
    assert np.array_equal(orc.matmul(F32, A, ne0, ne1, x, 2), (A.astype(np.float64) @ x.astype(np.float64)).astype(np.float32))


@pytest.mark.parametrize("mode", [0, 2])
def test_operators_against_float64(orc, rng, mode):
    x = (rng.standard_normal(1376) * 3).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 1376).astype(np.float32)
    assert rel(orc.rmsnorm(x, w, mode), np_ref.rmsnorm(x, w)) < 2e-6
    for hs, neox, base in ((64, 0, 1e4), (128, 0, 5e5), (96, 1, 1e4)):
        v = rng.standard_normal(hs * 3).astype(np.float32)
        for pos in (0, 1, 100, 4095):
            # the reference advances theta by repeated fp32 multiplication (src/inference.jl:126), so at
            # large positions the angle itself carries fp32 round-off: ~pos * 1e-7 absolute
            tol = 2e-6 + 4e-7 * pos
            assert rel(orc.rope(v, hs, 3, pos, base, neox, mode), np_ref.rope(v, hs, pos, base, neox)) < tol
    s = (rng.standard_normal(333) * 5).astype(np.float32)
    assert rel(orc.softmax(s, mode), np_ref.softmax(s)) < 2e-6
    a, b = (rng.standard_normal(500) * 4).astype(np.float32), rng.standard_normal(500).astype(np.float32)
    assert rel(orc.swiglu(a, b, mode), np_ref.swiglu(a, b)) < 2e-6
    for hs, nh, nkv, pos in ((64, 8, 8, 0), (128, 8, 2, 37), (96, 6, 6, 130), (64, 6, 2, 5)):
        q = rng.standard_normal(hs * nh).astype(np.float32)
        kc = rng.standard_normal((pos + 1, hs * nkv)).astype(np.float32)
        vc = rng.standard_normal((pos + 1, hs * nkv)).astype(np.float32)
        out, att = orc.attention(q, kc, vc, hs, nh, nkv, pos, mode)
        assert rel(out, np_ref.attention(q, kc, vc, hs, nh, nkv)) < 5e-6
        assert np.allclose(att.sum(1), 1, atol=1e-5)


def test_argmax_first_maximum(orc):
    assert orc.argmax(np.array([1, 5, 5, 2], np.float32)) == 1
    assert orc.argmax(np.array([-3, -1, -1], np.float32)) == 1
    assert orc.argmax(np.array([7], np.float32)) == 0


def _f32_model(rng, cfg):
    L, dim, hid = cfg["n_layers"], cfg["dim"], cfg["hidden_dim"]
    kv_dim = dim // cfg["n_heads"] * cfg["n_kv_heads"]
    g = lambda *s: (rng.standard_normal(s) * 0.05).astype(np.float32)
    W = dict(emb=g(cfg["vocab_size"], dim), output=g(cfg["vocab_size"], dim),
             rms_final=rng.uniform(0.8, 1.2, dim).astype(np.float32),
             rms_att=[rng.uniform(0.8, 1.2, dim).astype(np.float32) for _ in range(L)],
             rms_ffn=[rng.uniform(0.8, 1.2, dim).astype(np.float32) for _ in range(L)],
             wq=[g(dim, dim) for _ in range(L)], wk=[g(kv_dim, dim) for _ in range(L)],
             wv=[g(kv_dim, dim) for _ in range(L)], wo=[g(dim, dim) for _ in range(L)],
             w1=[g(hid, dim) for _ in range(L)], w2=[g(dim, hid) for _ in range(L)], w3=[g(hid, dim) for _ in range(L)])
    return W


@pytest.mark.parametrize("neox,n_kv", [(False, 4), (True, 2)])
def test_transformer_against_float64(orc, rng, neox, n_kv):
    """l2c_forward (layer order, residuals, KV cache, GQA head map, both RoPE styles) against a float64
    numpy transformer written from src/inference.jl:222-315."""
    cfg = dict(dim=64, hidden_dim=96, n_layers=3, n_heads=4, n_kv_heads=n_kv, vocab_size=50, seq_len=16,
               rope_freq_base=10000.0, rope_is_neox=neox)
    W = _f32_model(rng, cfg)
    T = {}
    def put(role, layer, a):
        a = np.ascontiguousarray(a, np.float32)
        T[(role, layer)] = (F32, a, a.shape[-1], 1 if a.ndim == 1 else a.shape[0])
    put(orc.TOK_EMB, 0, W["emb"]); put(orc.RMS_FINAL, 0, W["rms_final"]); put(orc.OUTPUT, 0, W["output"])
    for l in range(cfg["n_layers"]):
        for role, name in ((orc.RMS_ATT, "rms_att"), (orc.RMS_FFN, "rms_ffn"), (orc.WQ, "wq"), (orc.WK, "wk"),
                           (orc.WV, "wv"), (orc.WO, "wo"), (orc.W1, "w1"), (orc.W2, "w2"), (orc.W3, "w3")):
            put(role, l, W[name][l])
    m = orc.Model(cfg, T)
    tokens = [3, 17, 42, 8, 8, 1]
    want = np_ref.transformer_f32(cfg, W, tokens)
    for mode in (0, 2):
        m.reset()
        for pos, tok in enumerate(tokens):
            got = m.forward(tok, pos, mode)
            assert rel(got, want[pos]) < 2e-5, (mode, pos)
    # the greedy loop: prompt tokens are fed, then argmax (src/inference.jl:349-386)
    m.reset()
    ids, _ = m.generate_greedy(tokens[:3], 4, 2)
    seq = tokens[:3]
    for _ in range(4):
        seq = seq + [int(np.argmax(np_ref.transformer_f32(cfg, W, seq)[-1]))]
    assert ids.tolist() == seq[3:]


def test_q8k_half_way_cases_round_to_even(orc):
    """Round-half-to-even in l2c_quantize_q8_K, with expected bytes written by hand.  The block's extreme is
    -127, so iscale = -127 / -127 = 1 exactly and every other element x maps to rne(x): halves go to the
    even neighbour (0.5 -> 0, 1.5 -> 2, 2.5 -> 2, -0.5 -> 0, -1.5 -> -2, -2.5 -> -2, 126.5 -> 126), where
    round-half-away-from-zero would give 1, 2, 3, -1, -2, -3, 127.  With +127 as the extreme iscale is -1 and
    the signs flip; a value whose product lies just beside a half rounds to the nearer integer."""
    x = np.zeros(512, np.float32)
    vals = [-127.0, 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, -3.5, 126.5, -126.5, 0.49999997, 0.50000006, 1.0, -1.0, 63.5]
    want = [-127, 0, 2, 2, 4, 0, -2, -2, -4, 126, -126, 0, 1, 1, -1, 64]
    x[:16] = vals
    x[256:256 + 16] = [-v for v in vals]  # extreme +127: iscale = -1, q = rne(-x) = the same integers
    q = orc.quantize_q8_K(x)
    assert q[0]["qs"][:16].tolist() == want
    assert q[1]["qs"][:16].tolist() == want
    assert q[0]["d"] == 1.0 and q[1]["d"] == -1.0
    assert q[0]["bsums"][0] == sum(want) and not q[0]["qs"][16:].any()
    # the clamp: a product that rounds to 128 cannot occur (|x| <= |max|), but +127.5-like cases stay at 127
    y = np.zeros(256, np.float32)
    y[0], y[1] = -254.0, 253.5   # iscale = 0.5: 253.5 * 0.5 = 126.75 -> 127
    y[2] = 253.0                 # 126.5 -> 126 (half to even)
    y[3] = 251.0                 # 125.5 -> 126
    q = orc.quantize_q8_K(y)
    assert q[0]["qs"][:4].tolist() == [-127, 127, 126, 126]


def _quant_model(orc, rng, cfg, typ_layers, typ_out):
    """a small k-quant model: random blocks (valid by construction), returned as oracle tensors and as the
    float64-exact dequantized matrices of the same blocks"""
    dim, hid, L, V = cfg["dim"], cfg["hidden_dim"], cfg["n_layers"], cfg["vocab_size"]
    kv_dim = dim // cfg["n_heads"] * cfg["n_kv_heads"]
    T, W = {}, dict(rms_final=rng.uniform(0.8, 1.2, dim).astype(np.float32))

    def qmat(typ, rows, cols):
        raw = rand_blocks(rng, typ, rows * (cols // 256))
        return raw, np_ref.DEQUANT[typ](raw).reshape(rows, cols).astype(np.float32)

    def put(role, layer, typ, raw, ne0, ne1):
        T[(role, layer)] = (typ, raw, ne0, ne1)

    raw, W["emb"] = qmat(Q4, V, dim)
    put(orc.TOK_EMB, 0, Q4, raw, dim, V)
    raw, W["output"] = qmat(typ_out, V, dim)
    put(orc.OUTPUT, 0, typ_out, raw, dim, V)
    T[(orc.RMS_FINAL, 0)] = (F32, W["rms_final"], dim, 1)
    for name in ("rms_att", "rms_ffn", "wq", "wk", "wv", "wo", "w1", "w2", "w3"):
        W[name] = []
    shapes = dict(wq=(dim, dim), wk=(kv_dim, dim), wv=(kv_dim, dim), wo=(dim, dim), w1=(hid, dim), w2=(dim, hid),
                  w3=(hid, dim))
    roles = dict(wq=orc.WQ, wk=orc.WK, wv=orc.WV, wo=orc.WO, w1=orc.W1, w2=orc.W2, w3=orc.W3)
    for l in range(L):
        for name, role in (("rms_att", orc.RMS_ATT), ("rms_ffn", orc.RMS_FFN)):
            w = rng.uniform(0.8, 1.2, dim).astype(np.float32)
            W[name].append(w)
            T[(role, l)] = (F32, w, dim, 1)
        for name, (rows, cols) in shapes.items():
            raw, deq = qmat(typ_layers[name], rows, cols)
            W[name].append(deq)
            put(roles[name], l, typ_layers[name], raw, cols, rows)
    return T, W


@pytest.mark.parametrize("plan", ["q4", "q5_q6"])
def test_transformer_kquant_model_all_modes(orc, rng, plan):
    """l2c_forward on a k-quant model (the wiring of the quantized matvecs, and the embedding row of a token
    other than 0) against the float64 numpy transformer run on the dequantized matrices.  Mode 0 (float
    activations) must agree to fp32 round-off; modes 1 and 3 (q8_K activations) differ from it by the
    activation quantization step only, checked here as a bound far below what a wiring mistake (a swapped
    matrix, a wrong row offset, a missing residual) would cause."""
    cfg = dict(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=40, seq_len=8,
               rope_freq_base=10000.0, rope_is_neox=False)
    typ = dict.fromkeys(["wq", "wk", "wv", "wo", "w1", "w2", "w3"], Q4)
    out = Q4
    if plan == "q5_q6":
        typ = dict(typ, **dict.fromkeys(["wq", "wk", "wv", "wo", "w1", "w3"], Q5), w2=Q6)
        out = Q6
    T, W = _quant_model(orc, rng, cfg, typ, out)
    m = orc.Model(cfg, T)
    tokens = [7, 39, 1, 7]
    want = np_ref.transformer_f32(cfg, W, tokens)
    for mode, tol in ((0, 5e-6), (2, 1e-6), (1, 5e-2), (3, 5e-2)):  # observed 1.2e-6, 1e-7, 1e-2 to 3e-2; a wrong embedding row: 1.2e-1
        m.reset()
        for pos, tok in enumerate(tokens):
            got = m.forward(tok, pos, mode)
            assert rel(got, want[pos]) < tol, (plan, mode, pos, rel(got, want[pos]))
    # random blocks have scales of every size: the logits are large and structured, so a wiring mistake is
    # an O(1) difference; the q8_K modes stay within a few per cent of the float path and of each other
    m.reset()
    a = [m.forward(t, p, 1) for p, t in enumerate(tokens)]
    m.reset()
    b = [m.forward(t, p, 3) for p, t in enumerate(tokens)]
    for p in range(len(tokens)):
        assert rel(a[p], b[p]) < 1e-4  # fp32 against fp64 sums of the same integer dot products


def test_fp32_to_fp16_matches_numpy(orc, rng):
    """l2c_fp32_to_fp16 (the KV16 mode's rounding) against numpy's float16 conversion: random values over the
    whole range, every half-way point between consecutive half values and its two neighbours (ties go to even),
    the overflow threshold 65520, subnormals, zeros and infinities."""
    L = orc.lib()
    x = (rng.standard_normal(40000) * rng.choice([1e-8, 1e-5, 1e-3, 1, 100, 30000, 70000], 40000)).astype(np.float32)
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mid = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    edge = np.array([0, -0.0, 65504, 65519.996, 65520, 65536, 1e38, -1e38, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                     2.0 ** -25 * 1.0001, 2.0 ** -24 * 1.5, 2.0 ** -14, 2.0 ** -14 * (1 - 2.0 ** -11)], np.float32)
    x = np.concatenate([x, mid, -mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)), edge])
    got = np.array([L.l2c_fp32_to_fp16(float(v)) for v in x], np.uint16)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    back = np.array([L.l2c_fp16_to_fp32(int(b)) for b in got[:2000]], np.float32)
    assert np.array_equal(back, got[:2000].view(np.float16).astype(np.float32))

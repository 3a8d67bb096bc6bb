"""GPU parity of every operator of the decode path against the CPU oracle, through the C ABI.

Bars: bit-exact for the q8_K blocks, the per-block integer sums, dequantized weights, argmax
and the repacked weight bytes; floating point within the tolerance written in each test (the
HIP path and the oracle's L2C_CANON mode both round an fp64 sum once, so they normally agree to
the last bit; the tolerance only covers the fp64 summation order and the 1-ulp freedom of
exp/sin/cos).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q4, Q5, Q6, F32 = 12, 13, 14, 0


def _rel(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) / max(1e-30, np.max(np.abs(b))))


def _rand_blocks(rng, typ, n_blocks):
    """Random raw super-blocks with finite fp16 scales (every bit pattern of the integer fields)."""
    bb = {Q4: 144, Q5: 176, Q6: 210}[typ]
    raw = rng.integers(0, 256, size=(n_blocks, bb), dtype=np.uint8)
    d = rng.uniform(-0.01, 0.01, size=(n_blocks, 2)).astype(np.float16).view(np.uint8)
    if typ == Q6:
        raw[:, 208:210] = d[:, :2]
    else:
        raw[:, 0:4] = d
    return raw.reshape(-1)


@pytest.mark.parametrize("typ", [Q4, Q5, Q6])
def test_dequantize_bit_exact(pkg, orc, ctx, rng, typ):
    raw = _rand_blocks(rng, typ, 257)
    got = pkg.dequantize(raw, typ)
    want = orc.dequantize(typ, raw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def _q8_cases(rng):
    cases = {}
    cases["normal"] = rng.standard_normal(256 * 64).astype(np.float32)
    x = rng.standard_normal(256 * 4).astype(np.float32)
    x[256:512] = 0.0  # an all-zero block
    cases["zero_block"] = x
    x = rng.uniform(-1, 1, 256 * 8).astype(np.float32)
    for b in range(8):  # ties of the extreme: +m and -m at various places; the first one must win
        m = 1.5 + b
        i, j = sorted(rng.choice(256, 2, replace=False))
        x[256 * b + i] = m if b % 2 else -m
        x[256 * b + j] = -m if b % 2 else m
    cases["ties"] = x
    # the same with many blocks and with both holders inside one group of 16, in neighbouring groups, or far apart (the
    # streaming kernel's form of the quantizer searches a lane's 16 values by a tree and a block's 16 lanes by ballot)
    x = rng.uniform(-1, 1, 256 * 66).astype(np.float32)  # (66 blocks: the last group of four is half filled)
    for b in range(66):
        m = np.float32(2.0 + 0.25 * b)
        g = int(rng.integers(0, 16))
        if b % 3 == 0:
            i, j = sorted(rng.choice(16, 2, replace=False) + 16 * g)
        elif b % 3 == 1:
            i, j = 16 * g + int(rng.integers(0, 16)), 16 * ((g + 1) % 16) + int(rng.integers(0, 16))
            i, j = min(i, j), max(i, j)
        else:
            i, j = sorted(rng.choice(256, 2, replace=False))
        x[256 * b + i] = m if b % 2 else -m
        x[256 * b + j] = -m if b % 2 else m
        if b % 5 == 0:  # a third holder, later still
            k = int(rng.integers(j, 256))
            x[256 * b + k] = m
    cases["ties_many"] = x
    x = np.zeros(512, np.float32)
    x[:256] = (np.arange(256) - 127.5) / 127.0  # exact half-way products iscale*x = k + 0.5
    x[0] = -1.0
    x[256:] = np.float32(1e-38) * np.arange(256)  # the small ones are denormal
    cases["halfway_denormal"] = x
    cases["large"] = (rng.standard_normal(256 * 2) * 1e30).astype(np.float32)
    return cases


def test_quantize_q8k_bit_exact(pkg, orc, rng):
    for name, x in _q8_cases(rng).items():
        got = pkg.quantize_q8_K(x)
        want = orc.quantize_q8_K(x)
        assert got.tobytes() == want.tobytes(), name


def test_quantize_q8k_rejects_non_finite_input(pkg):
    """NaN or infinity in the input: an argument error, checked on the host before anything runs."""
    for bad in (np.nan, np.inf, -np.inf):
        x = np.ones(512, np.float32)
        x[300] = bad
        with pytest.raises(pkg.L2HError) as ei:
            pkg.quantize_q8_K(x)
        assert ei.value.code == -1 and "not finite" in str(ei.value)  # L2H_EINVAL


@pytest.mark.parametrize("typ", [Q4, Q5, Q6])
@pytest.mark.parametrize("ne0,ne1", [(256, 5), (768, 67), (4096, 130), (14336, 9)])
def test_matmul_kquant(pkg, orc, rng, typ, ne0, ne1):
    raw = _rand_blocks(rng, typ, ne1 * ne0 // 256)
    A = pkg.QuantMatrix(typ, raw, ne0, ne1)
    x = rng.standard_normal(ne0).astype(np.float32)
    y, isc, imin = pkg.matmul(A, x, return_ints=True)
    w_isc, w_imin = orc.matmul_ints(typ, raw, ne0, ne1, x)
    assert np.array_equal(isc, w_isc), "I_sc"
    assert np.array_equal(imin, w_imin), "I_min"
    want = orc.matmul(typ, raw, ne0, ne1, x, orc.GPU_SPEC)
    assert _rel(y, want) <= 1e-6  # fp64-accumulated on both sides
    y2 = pkg.matmul(A, x)  # the production (non-debug) kernel
    assert np.array_equal(y2.view(np.uint32), y.view(np.uint32))


@pytest.mark.parametrize("ne0,ne1", [(512, 33), (1376, 70), (30, 7)])
def test_matmul_f32(pkg, orc, rng, ne0, ne1):
    A = rng.standard_normal((ne1, ne0)).astype(np.float32)
    x = rng.standard_normal(ne0).astype(np.float32)
    y = pkg.matmul(A, x)
    want = orc.matmul(F32, A, ne0, ne1, x, orc.GPU_SPEC)
    assert _rel(y, want) <= 1e-6
    # against float64 numpy: the closed form
    assert _rel(y, (A.astype(np.float64) @ x.astype(np.float64)).astype(np.float32)) <= 1e-6


@pytest.mark.parametrize("typ", [Q4, Q5, Q6])
def test_weight_repack_round_trip(pkg, rng, typ):
    """The device layout is an exact permutation of the GGUF bytes."""
    from llama2_jl_amd import _lib, synth
    cfg = pkg.ModelConfig(dim=512, hidden_dim=768, n_layers=1, n_heads=4, n_kv_heads=4, vocab_size=64, seq_len=16)
    plan = dict(synth.PLAN_F32, w1=typ, wq=typ)
    lm = synth.synthetic_model(cfg, plan, seed=3)
    lm.weights.layers[0].w1 = pkg.QuantMatrix(typ, _rand_blocks(rng, typ, 768 * 2), 512, 768)
    dev = lm.device()
    for role, mat in ((_lib.W1, lm.weights.layers[0].w1), (_lib.WQ, lm.weights.layers[0].wq)):
        back = dev.get_tensor(role, 0, mat.data.size)
        assert np.array_equal(back, mat.data)


@pytest.mark.parametrize("n", [64, 512, 4096, 1376])
def test_rmsnorm(pkg, orc, ctx, rng, n):
    from llama2_jl_amd import _lib
    x = (rng.standard_normal(n) * 3).astype(np.float32)
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    o = np.empty(n, np.float32)
    ctx.check(_lib.lib().l2h_rmsnorm(ctx.handle, _lib.ptr(o), _lib.ptr(x), _lib.ptr(w), n))
    want = orc.rmsnorm(x, w, orc.GPU_SPEC)
    assert _rel(o, want) <= 1e-6
    x64 = x.astype(np.float64)
    closed = w * (x64 / np.sqrt(np.mean(x64 * x64) + 1e-5))
    assert _rel(o, closed.astype(np.float32)) <= 1e-5


@pytest.mark.parametrize("n", [256, 4096, 14336])
def test_rmsnorm_then_q8k_bit_exact(pkg, orc, ctx, rng, n):
    """The matvec prologue: rmsnorm then q8_K quantization, block for block."""
    from llama2_jl_amd import _lib, kquants
    x = (rng.standard_normal(n) * 2).astype(np.float32)
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    got = np.zeros(n // 256, kquants.block_q8_K)
    ctx.check(_lib.lib().l2h_rmsnorm_q8k(ctx.handle, _lib.ptr(x), _lib.ptr(w), n, _lib.ptr(got)))
    want = orc.quantize_q8_K(orc.rmsnorm(x, w, orc.GPU_SPEC))
    assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("hs,neox,base", [(64, 0, 10000.0), (128, 0, 500000.0), (96, 1, 10000.0)])
@pytest.mark.parametrize("pos", [0, 1, 17, 4095])
def test_rope(pkg, orc, ctx, rng, hs, neox, base, pos):
    from llama2_jl_amd import _lib
    n_heads = 5
    x = rng.standard_normal(hs * n_heads).astype(np.float32)
    got = x.copy()
    ctx.check(_lib.lib().l2h_rope(ctx.handle, _lib.ptr(got), hs, n_heads, pos, base, neox))
    want = orc.rope(x, hs, n_heads, pos, base, neox, orc.GPU_SPEC)
    assert _rel(got, want) <= 1e-6
    assert np.mean(got.view(np.uint32) != want.view(np.uint32)) < 0.01  # bit-equal but for rare 1-ulp cases


@pytest.mark.parametrize("n", [1, 7, 300, 4096])
def test_softmax(pkg, orc, ctx, rng, n):
    from llama2_jl_amd import _lib
    x = (rng.standard_normal(n) * 4).astype(np.float32)
    got = x.copy()
    ctx.check(_lib.lib().l2h_softmax(ctx.handle, _lib.ptr(got), n))
    want = orc.softmax(x, orc.GPU_SPEC)
    assert _rel(got, want) <= 1e-6
    assert abs(float(got.astype(np.float64).sum()) - 1.0) < 1e-5


@pytest.mark.parametrize("hs,n_heads,n_kv", [(64, 8, 8), (128, 32, 8), (96, 6, 6), (128, 4, 2), (64, 6, 2)])
@pytest.mark.parametrize("pos", [0, 5, 63, 64, 200])
def test_attention(pkg, orc, ctx, rng, hs, n_heads, n_kv, pos):
    from llama2_jl_amd import _lib
    q = rng.standard_normal(hs * n_heads).astype(np.float32)
    kc = rng.standard_normal((pos + 1, hs * n_kv)).astype(np.float32)
    vc = rng.standard_normal((pos + 1, hs * n_kv)).astype(np.float32)
    out = np.empty(hs * n_heads, np.float32)
    ctx.check(_lib.lib().l2h_attention(ctx.handle, _lib.ptr(out), _lib.ptr(q), _lib.ptr(kc), _lib.ptr(vc), hs, n_heads,
                                       n_kv, pos))
    want, _ = orc.attention(q, kc, vc, hs, n_heads, n_kv, pos, orc.GPU_SPEC)
    assert _rel(out, want) <= 2e-6


@pytest.mark.parametrize("hs,n_heads,n_kv,pos", [(96, 32, 32, 2047), (96, 32, 32, 2113), (96, 32, 32, 4000),
                                                 (128, 32, 8, 4000), (64, 6, 2, 1500), (128, 4, 2, 700)])
def test_attention_long_cache(pkg, orc, ctx, rng, hs, n_heads, n_kv, pos):
    """Caches of many 64-timestep tiles per head (scores, softmax and value sums in separate launches, the
    value sums split over the tiles); one row with scores far above the others'."""
    from llama2_jl_amd import _lib
    q = rng.standard_normal(hs * n_heads).astype(np.float32)
    kc = rng.standard_normal((pos + 1, hs * n_kv)).astype(np.float32)
    vc = rng.standard_normal((pos + 1, hs * n_kv)).astype(np.float32)
    kc[pos // 3] *= 3.0
    out = np.empty(hs * n_heads, np.float32)
    ctx.check(_lib.lib().l2h_attention(ctx.handle, _lib.ptr(out), _lib.ptr(q), _lib.ptr(kc), _lib.ptr(vc), hs, n_heads,
                                       n_kv, pos))
    want, _ = orc.attention(q, kc, vc, hs, n_heads, n_kv, pos, orc.GPU_SPEC)
    assert _rel(out, want) <= 2e-6


@pytest.mark.parametrize("hs,n_heads,n_kv,pos", [(72, 4, 2, 300), (40, 6, 3, 70), (256, 2, 1, 100), (8, 3, 3, 0)])
def test_attention_other_head_sizes(pkg, orc, ctx, rng, hs, n_heads, n_kv, pos):
    """Head sizes that are not a multiple of 16, or above 128: the general kernels (one lane per timestep
    for the scores, one thread per feature for the values)."""
    from llama2_jl_amd import _lib
    q = rng.standard_normal(hs * n_heads).astype(np.float32)
    kc = rng.standard_normal((pos + 1, hs * n_kv)).astype(np.float32)
    vc = rng.standard_normal((pos + 1, hs * n_kv)).astype(np.float32)
    out = np.empty(hs * n_heads, np.float32)
    ctx.check(_lib.lib().l2h_attention(ctx.handle, _lib.ptr(out), _lib.ptr(q), _lib.ptr(kc), _lib.ptr(vc), hs, n_heads,
                                       n_kv, pos))
    want, _ = orc.attention(q, kc, vc, hs, n_heads, n_kv, pos, orc.GPU_SPEC)
    assert _rel(out, want) <= 2e-6


def test_swiglu(pkg, orc, ctx, rng):
    from llama2_jl_amd import _lib
    n = 1376
    a = (rng.standard_normal(n) * 5).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    got = a.copy()
    ctx.check(_lib.lib().l2h_swiglu(ctx.handle, _lib.ptr(got), _lib.ptr(b), n))
    want = orc.swiglu(a, b, orc.GPU_SPEC)
    assert _rel(got, want) <= 1e-6


def test_argmax_first_maximum(pkg, orc, ctx, rng):
    import ctypes
    from llama2_jl_amd import _lib
    for n in (1, 5, 1000, 128256):
        x = rng.standard_normal(n).astype(np.float32)
        if n >= 5:
            m = x.max() + 1
            for i in sorted(rng.choice(n, 3, replace=False)):
                x[i] = m  # three equal maxima: the first index must be returned
        out = ctypes.c_int32(-1)
        ctx.check(_lib.lib().l2h_argmax(ctx.handle, _lib.ptr(x), n, ctypes.byref(out)))
        assert out.value == orc.argmax(x) == int(np.argmax(x))
    x = -np.abs(rng.standard_normal(100)).astype(np.float32) - 1  # all negative
    out = ctypes.c_int32(-1)
    ctx.check(_lib.lib().l2h_argmax(ctx.handle, _lib.ptr(x), 100, ctypes.byref(out)))
    assert out.value == int(np.argmax(x))


def test_error_paths(pkg, ctx, rng):
    """Bad arguments come back as error codes with a message; nothing is launched."""
    import ctypes
    from llama2_jl_amd import _lib
    x = np.zeros(100, np.float32)
    out = np.zeros(292, np.uint8)
    rc = _lib.lib().l2h_quantize_q8k(ctx.handle, _lib.ptr(x), 100, _lib.ptr(out))
    assert rc == _lib.EINVAL and b"256" in _lib.lib().l2h_last_error(ctx.handle)
    rc = _lib.lib().l2h_dequantize(ctx.handle, 2, _lib.ptr(out), 1, _lib.ptr(x))  # Q4_0: not implemented
    assert rc == _lib.ETYPE
    cfg = pkg.ModelConfig(dim=256, hidden_dim=256, n_layers=1, n_heads=2, n_kv_heads=2, vocab_size=8, seq_len=8)
    from llama2_jl_amd import synth
    lm = synth.synthetic_model(cfg, synth.PLAN_Q4_K, seed=1)
    lm.weights.layers[0].wq = np.zeros((128, 256), np.float32)  # wrong shape
    with pytest.raises(pkg.L2HError) as ei:
        lm.device()
    assert ei.value.code == _lib.EINVAL

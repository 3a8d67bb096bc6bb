"""Batched prompt pass (l2h_prefill) against the CPU oracle's per-token loop.

The reference has no batched path: the result is defined as what transformer! leaves behind when
called for each position in turn (src/inference.jl:222-315).  The device computes the matrix products
in bf16 on the matrix cores (float activations, no q8_K step), so the comparison is against the
oracle's float-activation mode with a tolerance for bf16 rounding: relative max-abs error of the K/V
cache rows <= 2e-2 and of the last position's logits <= 3e-2 (observed values are printed).
"""
import numpy as np
import pytest

from test_gpu_model import CASES, _model, _rel

pytestmark = pytest.mark.gpu

KV_TOL, LOGIT_TOL = 2e-2, 3e-2


def _oracle_run(orc, om, tokens, pos0=0):
    logits = None
    for i, t in enumerate(tokens):
        logits = om.forward(int(t), pos0 + i, orc.CANON)
    return logits


@pytest.mark.parametrize("library", [True, False], ids=["library_products", "own_products"])
@pytest.mark.parametrize("case", sorted(CASES))
def test_prefill_matches_token_loop(pkg, orc, case, library):
    """library: the plain products (q|k|v, wo, w2) through hipBLASLt (the default) or through this library's kernels."""
    from llama2_jl_amd import synth
    plan, kw = CASES[case]
    lm = _model(pkg, plan, **kw)
    cfg = lm.config
    n1, n2 = 45, cfg.seq_len - 45 - 9  # two calls: positions 0..44, then 45.. (queries see earlier keys)
    prompt = synth.seeded_prompt(21, n1 + n2, cfg.vocab_size)
    dev = lm.device()
    dev.set_prefill_library(library)
    om = orc.model_from_language_model(lm, nthreads=8)
    dev.reset()
    om.reset()
    logits, nxt = dev.prefill(prompt[:n1], 0)
    # (the library takes over where the bf16 copy exists: dim and hidden_dim multiples of 64)
    assert dev.prefill_library == (library and cfg.dim % 64 == 0 and cfg.hidden_dim % 64 == 0)
    ref = _oracle_run(orc, om, prompt[:n1])
    e1 = _rel(logits, ref)
    assert nxt == int(np.argmax(logits))
    logits, nxt = dev.prefill(prompt[n1:], n1)
    ref = _oracle_run(orc, om, prompt[n1:], n1)
    e2 = _rel(logits, ref)
    ekv = 0.0
    for layer in range(cfg.n_layers):
        k, v = dev.kv_read(layer, 0, n1 + n2)
        rk, rv = om.kv_read(layer, 0, n1 + n2)
        ekv = max(ekv, _rel(k, rk), _rel(v, rv))
    print("\n[%s, %s] prefill vs token loop: logits rel err %.3g / %.3g, K/V rel err %.3g"
          % (case, "hipBLASLt products" if dev.prefill_library else "own products", e1, e2, ekv))
    assert e1 <= LOGIT_TOL and e2 <= LOGIT_TOL and ekv <= KV_TOL
    # decoding continues from the cache the prompt pass left
    ids = dev.generate_greedy([nxt], 4, pos0=n1 + n2)
    assert len(ids) == 4


def test_prefill_then_decode_matches_decode_only(pkg):
    """The cache written by the prompt pass is the cache the per-token path would have written, to
    bf16 accuracy: the next-token logits of a decode step on top of either agree within tolerance."""
    from llama2_jl_amd import synth
    plan, kw = CASES["q4ks_gqa"]
    lm = _model(pkg, plan, **kw)
    prompt = synth.seeded_prompt(3, 100, kw["vocab_size"])
    dev = lm.device()
    dev.reset()
    _, l_seq = dev.generate_greedy(prompt, 1, want_logits=True)
    dev.reset()
    dev.prefill(prompt[:-1], 0, want_logits=False)
    l_pf, _ = dev.forward(int(prompt[-1]), len(prompt) - 1)
    err = _rel(l_pf, l_seq)
    print("\nprefill+decode vs decode-only (q8_K path): logits rel diff %.3g" % err)
    assert err <= 5e-2  # bf16 prompt pass vs q8_K per-token pass: two different roundings of the same sum


# a wider model than CASES holds: many K steps per product, several position tiles, the last one part filled
WIDE = ("PLAN_Q5_K_M", dict(dim=512, hidden_dim=1536, n_layers=2, n_heads=8, n_kv_heads=4, vocab_size=512, seq_len=330,
                            rope_freq_base=10000.0, rope_is_neox=False))


# w1|w3 with 86 groups of 256 rows at 300 positions: more than one round of 256 x 128 tiles on 256 CUs, less than
# one of 256 x 256 ones, which is where the product kernel mixes the two tile shapes in one launch
MIXED = ("PLAN_F32", dict(dim=64, hidden_dim=11008, n_layers=1, n_heads=2, n_kv_heads=2, vocab_size=512, seq_len=303,
                          rope_freq_base=10000.0, rope_is_neox=False))


@pytest.mark.parametrize("case", sorted(CASES) + ["wide", "mixed"])
def test_prefill_weight_copy_changes_nothing(pkg, case):
    """l2h_prefill multiplies from a resident bf16 copy of the weights (default) or expands the quantized
    blocks inside the product kernel (l2h_model_set_prefill_copy(m, 0)): the same bf16 values either way,
    so with this library's own product kernels logits and cache are equal bit for bit.  With the plain products
    through hipBLASLt (the default) the same sums are formed in another order: equal to fp32 rounding per product, which
    the next rounding of an activation to bf16 turns into a difference of bf16 size for the odd element."""
    from llama2_jl_amd import synth
    plan, kw = WIDE if case == "wide" else MIXED if case == "mixed" else CASES[case]
    lm = _model(pkg, plan, **kw)
    cfg = lm.config
    n = cfg.seq_len - 3
    prompt = synth.seeded_prompt(8, n, cfg.vocab_size)
    dev = lm.device()
    dev.set_prefill_library(False)
    got = []
    for on in (True, False, True):
        dev.set_prefill_copy(on)
        dev.reset()
        logits, nxt = dev.prefill(prompt, 0)
        assert not dev.prefill_library
        k, v = dev.kv_read(cfg.n_layers - 1, 0, n)
        got.append((logits.copy(), nxt, k.copy(), v.copy()))
    dev.set_prefill_copy(True)
    for other in got[1:]:
        assert other[1] == got[0][1]
        assert np.array_equal(other[0], got[0][0])
        assert np.array_equal(other[2], got[0][2]) and np.array_equal(other[3], got[0][3])
    # the library's products on the same copy (its three matrices rewritten as plain rows), and back again
    dev.set_prefill_library(True)
    dev.reset()
    logits, nxt = dev.prefill(prompt, 0)
    if cfg.dim % 64 == 0 and cfg.hidden_dim % 64 == 0:
        assert dev.prefill_library
    k, v = dev.kv_read(cfg.n_layers - 1, 0, n)
    e, ekv = _rel(logits, got[0][0]), max(_rel(k, got[0][2]), _rel(v, got[0][3]))
    print("\n[%s] hipBLASLt products against own products: logits rel diff %.3g, K/V rel diff %.3g" % (case, e, ekv))
    # (the products agree to fp32 rounding -- the first layer's K/V rows are equal -- but a difference in the last bit of the
    # residual stream now and then turns a rounding to bf16 the other way: a few per mille of the affected rows' values)
    assert e <= 1.5e-2 and ekv <= 1e-2
    dev.set_prefill_library(False)
    dev.reset()
    logits, nxt = dev.prefill(prompt, 0)
    assert not dev.prefill_library and nxt == got[0][1] and np.array_equal(logits, got[0][0])


def test_prefill_without_the_gemm_library(pkg, monkeypatch):
    """Where hipBLASLt cannot be opened (here: L2H_HIPBLASLT names a file that does not exist) the prompt pass runs this
    library's product kernels and says so; same results, bit for bit, as with the library switched off by the caller."""
    from llama2_jl_amd import synth
    plan, kw = CASES["q4ks_gqa"]
    lm = _model(pkg, plan, **kw)
    prompt = synth.seeded_prompt(5, lm.config.seq_len - 7, lm.config.vocab_size)
    got = []
    for missing in (True, False):
        if missing:
            monkeypatch.setenv("L2H_HIPBLASLT", "/nonexistent/libhipblaslt.so")
        else:
            monkeypatch.delenv("L2H_HIPBLASLT", raising=False)
        lm._device = None
        dev = lm.device()
        if not missing:
            dev.set_prefill_library(False)
        logits, nxt = dev.prefill(prompt, 0)
        assert not dev.prefill_library
        got.append((logits.copy(), nxt))
        dev.close()
    assert got[0][1] == got[1][1] and np.array_equal(got[0][0], got[1][0])


def test_prefill_with_a_gemm_library_that_has_no_algorithm(pkg, monkeypatch):
    """The library opens but offers nothing for the products (L2H_PF_LT_CANDIDATES=0 stands for an installation without
    the kernels for this device): noticed before anything is computed with it, the own product kernels take over and the
    copy's matrices are rewritten as tiles; same results, bit for bit, as with the library switched off."""
    from llama2_jl_amd import synth
    plan, kw = CASES["q5km"]
    lm = _model(pkg, plan, **kw)
    prompt = synth.seeded_prompt(6, lm.config.seq_len - 5, lm.config.vocab_size)
    got = []
    for none in (True, False):
        if none:
            monkeypatch.setenv("L2H_PF_LT_CANDIDATES", "0")
        else:
            monkeypatch.delenv("L2H_PF_LT_CANDIDATES", raising=False)
        lm._device = None
        dev = lm.device()
        if not none:
            dev.set_prefill_library(False)
        for rep in range(2):  # (the second call finds the library already given up)
            dev.reset()
            logits, nxt = dev.prefill(prompt, 0)
            assert not dev.prefill_library
            got.append((logits.copy(), nxt))
        dev.close()
    for other in got[1:]:
        assert other[1] == got[0][1] and np.array_equal(other[0], got[0][0])


def test_prefill_longer_than_one_chunk(pkg, orc):
    """More positions than one internal chunk (2048): the second chunk's queries attend to the first's keys."""
    from llama2_jl_amd import synth
    kw = dict(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=300, seq_len=2200,
              rope_freq_base=10000.0, rope_is_neox=False)
    lm = _model(pkg, "PLAN_Q4_K_S", **kw)
    prompt = synth.seeded_prompt(4, 2100, kw["vocab_size"])
    dev = lm.device()
    om = orc.model_from_language_model(lm, nthreads=8)
    dev.reset()
    om.reset()
    logits, nxt = dev.prefill(prompt, 0)
    ref = _oracle_run(orc, om, prompt)
    err = _rel(logits, ref)
    k, v = dev.kv_read(1, 2040, 60)
    rk, rv = om.kv_read(1, 2040, 60)
    print("\n2100-position prompt: logits rel err %.3g, last K/V rows %.3g" % (err, max(_rel(k, rk), _rel(v, rv))))
    assert err <= LOGIT_TOL and _rel(k, rk) <= KV_TOL and _rel(v, rv) <= KV_TOL


def test_prefill_headline_widths_against_token_loop(pkg, orc):
    """The prompt pass at the headline's widths (dim 4096, hidden 14336, 32 / 8 heads of 128, q4_K layers; K = 4096 and
    14336 in the products), two layers deep and with a small vocabulary so that the oracle's token loop finishes in
    seconds, 320 positions (w1|w3 then runs as the launch that mixes 256 x 256 and 256 x 128 tiles): every layer's K/V
    rows and the last logits against the oracle, at the same tolerances as the small shapes; with and without the
    bf16 weight copy."""
    from llama2_jl_amd import synth
    kw = dict(dim=4096, hidden_dim=14336, n_layers=2, n_heads=32, n_kv_heads=8, vocab_size=2048, seq_len=336,
              rope_freq_base=500000.0, rope_is_neox=False)
    lm = _model(pkg, "PLAN_Q4_K_S", **kw)
    n = 320
    prompt = synth.seeded_prompt(13, n, kw["vocab_size"])
    om = orc.model_from_language_model(lm, nthreads=16)
    om.reset()
    ref = _oracle_run(orc, om, prompt)
    dev = lm.device()
    for on in (True, False):
        dev.set_prefill_copy(on)
        dev.reset()
        logits, nxt = dev.prefill(prompt, 0)
        e = _rel(logits, ref)
        ekv = 0.0
        for layer in range(2):
            k, v = dev.kv_read(layer, 0, n)
            rk, rv = om.kv_read(layer, 0, n)
            ekv = max(ekv, _rel(k, rk), _rel(v, rv))
        print("\n[headline widths, bf16 copy %s] prefill vs token loop: logits rel err %.3g, K/V rel err %.3g" % (on, e, ekv))
        assert e <= LOGIT_TOL and ekv <= KV_TOL
    dev.set_prefill_copy(True)
    dev.close()
    om.close()


def test_prefill_argument_checks(pkg):
    plan, kw = CASES["f32"]
    lm = _model(pkg, plan, **kw)
    dev = lm.device()
    with pytest.raises(pkg.L2HError):
        dev.prefill(np.zeros(0, np.int32), 0)
    with pytest.raises(pkg.L2HError):
        dev.prefill([1, 2, 3], lm.config.seq_len - 2)
    with pytest.raises(pkg.L2HError):
        dev.prefill([lm.config.vocab_size], 0)
    # l2h_model_set_prefill_copy takes 0 or 1
    from llama2_jl_amd import _lib
    assert _lib.lib().l2h_model_set_prefill_copy(dev.handle, 2) != 0
    assert _lib.lib().l2h_model_set_prefill_copy(dev.handle, 1) == 0

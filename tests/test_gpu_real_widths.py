"""The benchmark configurations at their real widths against the CPU oracle.

The small shapes of test_gpu_model.py never reach 12 or 32 super-blocks per row, head size 96 next to
a 4096-long cache, or an fp32 model of the llama2.c size.  Here every configuration runs at the widths
the benchmark uses: two layers deep where 128 tokens are compared (the oracle then finishes in
seconds), all 32 layers where a handful of tokens are (the oracle follows a full-size model at a few
tokens per second).  Bar: greedy tokens identical to the oracle in the mode the HIP path implements
(q8_K activations for k-quant weights, fp64 sums), final logits within 1e-3 relative max-abs.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) / max(1e-30, np.max(np.abs(b))))


def _model(pkg, plan_name, seed, **kw):
    from llama2_jl_amd import synth
    cfg = pkg.ModelConfig(**kw)
    return synth.synthetic_model(cfg, getattr(synth, plan_name), seed=seed, share_classifier=(plan_name == "PLAN_F32"))


def _prefill_rows(dev, om, cfg, n_pre, seed):
    """seeded random K/V rows for positions 0..n_pre-1 of every layer, on both sides"""
    rng = np.random.default_rng(seed)
    kv_dim = cfg.dim // cfg.n_heads * cfg.n_kv_heads
    for layer in range(cfg.n_layers):
        kv = rng.standard_normal((2, n_pre, kv_dim), dtype=np.float32)
        dev.kv_write(layer, 0, kv[0], kv[1])
        om.kv_write(layer, 0, kv[0], kv[1])


def test_llama2c_fp32_full_size(pkg, orc):
    """Configuration 1 as it is: the llama2.c stories-42M shape (reference src/load_karpathy.jl:1-59), fp32
    weights, classifier shared with the embedding, 16-token prompt, 256 greedy tokens."""
    from llama2_jl_amd import synth
    kw = dict(dim=512, hidden_dim=1376, n_layers=8, n_heads=8, n_kv_heads=8, vocab_size=32000, seq_len=1024,
              rope_freq_base=10000.0, rope_is_neox=False)
    lm = _model(pkg, "PLAN_F32", 31, **kw)
    prompt = synth.seeded_prompt(16, 16, kw["vocab_size"])
    dev = lm.device()
    om = orc.model_from_language_model(lm, nthreads=16)
    ids, logits = dev.generate_greedy(prompt, 256, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy(prompt, 256, orc.GPU_SPEC)
    print("\n[llama2c fp32, full size] logits rel err %.3g" % _rel(logits, ref_logits))
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    dev.close()
    om.close()


@pytest.mark.parametrize("path", [0, 1])
def test_phi3_widths_long_cache(pkg, orc, path):
    """Configuration 4's widths, two layers: dim 3072 (12 super-blocks per row), hidden 8192 (32), 32 heads
    of 96 without GQA, neox RoPE, vocabulary 32064, a 4096-long cache whose first 3840 rows are seeded
    random numbers written through l2h_kv_write; 16 greedy tokens from position 3840.  path 0 = the
    library's own choice of launch path, 1 = one kernel per phase."""
    kw = dict(dim=3072, hidden_dim=8192, n_layers=2, n_heads=32, n_kv_heads=32, vocab_size=32064, seq_len=4096,
              rope_freq_base=10000.0, rope_is_neox=True)
    lm = _model(pkg, "PLAN_Q4_K", 32, **kw)
    dev = lm.device(path=path)
    om = orc.model_from_language_model(lm, nthreads=16)
    _prefill_rows(dev, om, lm.config, 3840, 4)
    ids, logits = dev.generate_greedy([11], 16, pos0=3840, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy([11], 16, orc.GPU_SPEC, pos0=3840)
    print("\n[phi3 widths, launch path %d] logits rel err %.3g" % (dev.path, _rel(logits, ref_logits)))
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    dev.close()
    om.close()


@pytest.mark.parametrize("path", [0, 1])
def test_q5km_headline_widths(pkg, orc, path):
    """Configuration 3's tensor types (q5_K attention and up/gate, q6_K down and output) at the 8B widths
    (dim 4096, hidden 14336, 32/8 heads of 128), two layers: 128 greedy tokens from a 32-token prompt."""
    from llama2_jl_amd import synth
    kw = dict(dim=4096, hidden_dim=14336, n_layers=2, n_heads=32, n_kv_heads=8, vocab_size=32000, seq_len=192,
              rope_freq_base=500000.0, rope_is_neox=False)
    lm = _model(pkg, "PLAN_Q5_K_M", 33, **kw)
    prompt = synth.seeded_prompt(99, 32, kw["vocab_size"])
    dev = lm.device(path=path)
    om = orc.model_from_language_model(lm, nthreads=16)
    ids, logits = dev.generate_greedy(prompt, 128, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy(prompt, 128, orc.GPU_SPEC)
    print("\n[q5_K_M, 8B widths, launch path %d] logits rel err %.3g" % (dev.path, _rel(logits, ref_logits)))
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    dev.close()
    om.close()


def test_q5km_full_size_against_oracle(pkg, orc):
    """Configuration 3 at its full size (32 layers, vocabulary 128256): the oracle follows it for a 4-token
    prompt and 6 greedy tokens; then the library's choice of launch path against one kernel per phase over the
    benchmark's 128 tokens, bit for bit."""
    from llama2_jl_amd import synth
    kw = dict(dim=4096, hidden_dim=14336, n_layers=32, n_heads=32, n_kv_heads=8, vocab_size=128256, seq_len=512,
              rope_freq_base=500000.0, rope_is_neox=False)
    lm = _model(pkg, "PLAN_Q5_K_M", 34, **kw)
    prompt = synth.seeded_prompt(5, 4, kw["vocab_size"])
    dev = lm.device()
    om = orc.model_from_language_model(lm, nthreads=16)
    ids, logits = dev.generate_greedy(prompt, 6, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy(prompt, 6, orc.GPU_SPEC)
    om.close()
    print("\n[q5_K_M, full size, launch path %d] logits rel err %.3g" % (dev.path, _rel(logits, ref_logits)))
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    long_prompt = synth.seeded_prompt(7, 32, kw["vocab_size"])
    dev.reset()
    a_ids, a_logits = dev.generate_greedy(long_prompt, 128, want_logits=True)
    a_path = dev.path
    dev.close()
    other = 2 if a_path == 1 else 1
    dev2 = lm.device(path=other)
    b_ids, b_logits = dev2.generate_greedy(long_prompt, 128, want_logits=True)
    dev2.close()
    assert np.asarray(a_ids).tolist() == np.asarray(b_ids).tolist()
    assert np.array_equal(a_logits.view(np.uint32), b_logits.view(np.uint32))


def test_q4ks_full_size_against_oracle(pkg, orc):
    """Configuration 2, the headline, at its full size (32 layers, vocabulary 128256, q4_K layers, q6_K output): the
    oracle follows it for a 4-token prompt and 6 greedy tokens on the library's own choice of launch path (the
    streaming kernel)."""
    from llama2_jl_amd import synth
    kw = dict(dim=4096, hidden_dim=14336, n_layers=32, n_heads=32, n_kv_heads=8, vocab_size=128256, seq_len=512,
              rope_freq_base=500000.0, rope_is_neox=False)
    lm = _model(pkg, "PLAN_Q4_K_S", 35, **kw)
    prompt = synth.seeded_prompt(6, 4, kw["vocab_size"])
    dev = lm.device()
    assert dev.path == 3
    om = orc.model_from_language_model(lm, nthreads=16)
    ids, logits = dev.generate_greedy(prompt, 6, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy(prompt, 6, orc.GPU_SPEC)
    print("\n[Q4_K_S, full size, launch path 3] logits rel err %.3g" % _rel(logits, ref_logits))
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    # How far the q8_K step moves a random-weight model of this depth, for scale (the prompt pass multiplies float
    # activations, and tests/test_gpu_model.py compares it with sequential decode at this size): the oracle's two
    # arithmetics fed the same nine tokens, logits at the last position.
    fed = list(prompt) + [int(t) for t in ref_ids[:5]]
    last = {}
    for mode in (orc.GPU_SPEC, orc.REFERENCE):
        om.reset()
        for pos, tok in enumerate(fed):
            last[mode] = om.forward(int(tok), pos, mode)
    a, b = last[orc.GPU_SPEC].astype(np.float64), last[orc.REFERENCE].astype(np.float64)
    rms = float(np.sqrt(np.mean((a - b) ** 2)) / np.sqrt(np.mean(b ** 2)))
    print("[Q4_K_S, full size] oracle with q8_K activations vs with float activations, 32 layers, position 8: logits rel "
          "diff max %.3g, rms %.3g" % (_rel(last[orc.GPU_SPEC], last[orc.REFERENCE]), rms))
    om.close()
    dev.close()


def test_phi3_full_size_against_oracle(pkg, orc):
    """Configuration 4 at its full size (32 layers) with its 4096-long cache, 3840 rows pre-filled: six greedy
    tokens from position 3840 against the oracle."""
    kw = dict(dim=3072, hidden_dim=8192, n_layers=32, n_heads=32, n_kv_heads=32, vocab_size=32064, seq_len=4096,
              rope_freq_base=10000.0, rope_is_neox=True)
    lm = _model(pkg, "PLAN_Q4_K", 35, **kw)
    dev = lm.device()
    om = orc.model_from_language_model(lm, nthreads=16)
    _prefill_rows(dev, om, lm.config, 3840, 9)
    ids, logits = dev.generate_greedy([11], 6, pos0=3840, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy([11], 6, orc.GPU_SPEC, pos0=3840)
    print("\n[phi3, full size, launch path %d] logits rel err %.3g" % (dev.path, _rel(logits, ref_logits)))
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    dev.close()
    om.close()


def test_q4ks_file_mix_runs_on_the_streaming_kernel(pkg, orc):
    """The tensor mix a Q4_K_S file is said to carry (q5_K attn_v and ffn_down in the first layers) at the 8B widths,
    two layers of which the first holds the q5_K tensors: the streaming kernel takes it with typed pieces (q4_K and
    q5_K rows next to each other in the q|k|v phase).  128 greedy tokens against the oracle, and the per-phase path
    bit for bit.  A model the kernel cannot take (dim 1024: rows are half a piece) falls to one kernel per
    phase and says why."""
    from llama2_jl_amd import synth
    kw = dict(dim=4096, hidden_dim=14336, n_layers=2, n_heads=32, n_kv_heads=8, vocab_size=32000, seq_len=192,
              rope_freq_base=500000.0, rope_is_neox=False)
    cfg = pkg.ModelConfig(**kw)
    lm = synth.synthetic_model(cfg, synth.plan_q4_k_s_file(2, n_first=1), seed=36)
    assert lm.weights.layers[0].wv.type == 13 and lm.weights.layers[0].w2.type == 13 and lm.weights.layers[1].wv.type == 12
    prompt = synth.seeded_prompt(99, 32, kw["vocab_size"])
    dev = lm.device()
    assert dev.path == 3 and dev.path_reason == ""
    om = orc.model_from_language_model(lm, nthreads=16)
    ids, logits = dev.generate_greedy(prompt, 128, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy(prompt, 128, orc.GPU_SPEC)
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    dev.close()
    om.close()
    dev1 = lm.device(path=1)
    ids1, logits1 = dev1.generate_greedy(prompt, 128, want_logits=True)
    dev1.close()
    assert ids1.tolist() == ids.tolist()
    assert np.array_equal(logits1.view(np.uint32), logits.view(np.uint32))
    lm3 = _model(pkg, "PLAN_Q4_K", 37, **dict(kw, dim=1024, hidden_dim=4096, n_heads=8, n_kv_heads=8, n_layers=1,
                                              vocab_size=1000))
    dev3 = lm3.device()
    assert dev3.path == 1 and "2048" in dev3.path_reason
    dev3.close()

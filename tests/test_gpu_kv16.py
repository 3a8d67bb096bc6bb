"""The optional fp16 KV cache (l2h_model_set_kv_type) against the oracle with the same rounding.

The reference's cache is Float32 (src/inference.jl:62-70) and stays the default; the fp16 cache halves the
bytes a decode step reads from it.  Specification: a row is rounded to binary16 (nearest even) when it is
appended and widened exactly when it is read; nothing else changes.  The oracle does the same under its KV16
mode bit (its rounding routine is pinned against numpy's float16 conversion in tests/test_oracle.py), so the
bar is the usual one: identical greedy tokens, logits within 1e-3 relative max-abs (observed: identical)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) / max(1e-30, np.max(np.abs(b))))


def _model(pkg, plan, **kw):
    from llama2_jl_amd import synth
    return synth.synthetic_model(pkg.ModelConfig(**kw), getattr(synth, plan), seed=kw["dim"] + 3,
                                 share_classifier=(plan == "PLAN_F32"))


CASES = {
    "q4ks_gqa_hs128": ("PLAN_Q4_K_S", dict(dim=512, hidden_dim=1024, n_layers=3, n_heads=4, n_kv_heads=1, vocab_size=1000,
                                           seq_len=160, rope_freq_base=500000.0, rope_is_neox=False)),
    "phi3_hs96": ("PLAN_Q4_K", dict(dim=768, hidden_dim=1024, n_layers=2, n_heads=8, n_kv_heads=8, vocab_size=512,
                                    seq_len=128, rope_freq_base=10000.0, rope_is_neox=True)),
    "f32_hs32": ("PLAN_F32", dict(dim=128, hidden_dim=344, n_layers=3, n_heads=4, n_kv_heads=2, vocab_size=500, seq_len=96,
                                  rope_freq_base=10000.0, rope_is_neox=False)),
    "q5km_long": ("PLAN_Q5_K_M", dict(dim=512, hidden_dim=768, n_layers=2, n_heads=8, n_kv_heads=2, vocab_size=600,
                                      seq_len=1280, rope_freq_base=10000.0, rope_is_neox=False)),
    # shapes that the streaming kernel takes (launch path 3): its long-cache attention reads the fp16 cache at every
    # position; head sizes 128 with GQA, 96 (the Phi-3 widths) and 64
    "flow_q4_hs128": ("PLAN_Q4_K", dict(dim=2048, hidden_dim=2048, n_layers=2, n_heads=16, n_kv_heads=4, vocab_size=600,
                                        seq_len=128, rope_freq_base=500000.0, rope_is_neox=False)),
    "flow_phi3_hs96": ("PLAN_Q4_K", dict(dim=3072, hidden_dim=2048, n_layers=2, n_heads=32, n_kv_heads=32, vocab_size=512,
                                         seq_len=128, rope_freq_base=10000.0, rope_is_neox=True)),
    "flow_q5km_hs64": ("PLAN_Q5_K_M", dict(dim=4096, hidden_dim=2048, n_layers=2, n_heads=64, n_kv_heads=16, vocab_size=600,
                                           seq_len=128, rope_freq_base=10000.0, rope_is_neox=False)),
}


@pytest.mark.parametrize("case", sorted(CASES))
def test_fp16_cache_matches_oracle(pkg, orc, case):
    from llama2_jl_amd import synth
    plan, kw = CASES[case]
    lm = _model(pkg, plan, **kw)
    cfg = lm.config
    dev = lm.device(kv_fp16=True)
    assert dev.path == (3 if case.startswith("flow_") else 1)
    om = orc.model_from_language_model(lm, nthreads=16)
    mode = orc.GPU_SPEC | orc.KV16
    prompt = synth.seeded_prompt(5, 6, cfg.vocab_size)
    ids, logits = dev.generate_greedy(prompt, 40, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy(prompt, 40, mode)
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    # the cache rows are the oracle's (fp16 values, widened)
    for layer in range(cfg.n_layers):
        k, v = dev.kv_read(layer, 0, 45)
        rk, rv = om.kv_read(layer, 0, 45)
        assert np.array_equal(k, rk) and np.array_equal(v, rv)
        assert np.array_equal(k, k.astype(np.float16).astype(np.float32))
    # against the same model with the reference's fp32 cache: close, and reported
    om.reset()
    f_ids, f_logits = om.generate_greedy(prompt, 40, orc.GPU_SPEC)
    same = int(np.argmax(np.append(ids != f_ids, True)))
    print("\n[%s] fp16 cache: logits rel err vs oracle(KV16) %.3g; first %d of 40 greedy tokens equal to the fp32 cache's"
          % (case, _rel(logits, ref_logits), same))
    dev.close()
    om.close()


def test_fp16_cache_prefilled_long(pkg, orc, rng):
    """l2h_kv_write into an fp16 cache rounds the rows (returned so by l2h_kv_read); decoding on top of 1100
    pre-filled positions, several attention tiles and two softmax workgroups deep."""
    plan, kw = CASES["phi3_hs96"]
    kw = dict(kw, seq_len=1300)
    lm = _model(pkg, plan, **kw)
    cfg = lm.config
    dev = lm.device(kv_fp16=True)
    om = orc.model_from_language_model(lm, nthreads=8)
    kv_dim = cfg.dim // cfg.n_heads * cfg.n_kv_heads
    n_pre = 1100
    for layer in range(cfg.n_layers):
        k = rng.standard_normal((n_pre, kv_dim)).astype(np.float32)
        v = (rng.standard_normal((n_pre, kv_dim)) * 3).astype(np.float32)
        dev.kv_write(layer, 0, k, v)
        k16, v16 = k.astype(np.float16).astype(np.float32), v.astype(np.float16).astype(np.float32)
        om.kv_write(layer, 0, k16, v16)
        k2, v2 = dev.kv_read(layer, 0, n_pre)
        assert np.array_equal(k2, k16) and np.array_equal(v2, v16)
    ids, logits = dev.generate_greedy([7], 12, pos0=n_pre, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy([7], 12, orc.GPU_SPEC | orc.KV16, pos0=n_pre)
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    dev.close()
    om.close()


def test_fp16_cache_limits(pkg):
    from llama2_jl_amd import synth
    from llama2_jl_amd.inference import DeviceModel
    plan, kw = "PLAN_Q4_K", dict(dim=2048, hidden_dim=2048, n_layers=1, n_heads=16, n_kv_heads=4, vocab_size=300,
                                 seq_len=64, rope_freq_base=10000.0, rope_is_neox=False)
    lm = _model(pkg, plan, **kw)
    with pytest.raises(pkg.L2HError):  # the persistent kernel with grid barriers reads fp32 caches
        DeviceModel(lm.config, lm.weights, path=2, kv_fp16=True)
    dev = DeviceModel(lm.config, lm.weights, kv_fp16=True)  # automatic choice: the streaming kernel
    assert dev.path == 3
    with pytest.raises(pkg.L2HError):  # the batched prompt pass writes an fp32 cache
        dev.prefill(synth.seeded_prompt(1, 8, 300), 0)
    dev.close()
    # head size 20: neither a multiple of 16
    lm2 = _model(pkg, "PLAN_F32", dim=80, hidden_dim=96, n_layers=1, n_heads=4, n_kv_heads=4, vocab_size=50, seq_len=32,
                 rope_freq_base=10000.0, rope_is_neox=False)
    with pytest.raises(pkg.L2HError):
        DeviceModel(lm2.config, lm2.weights, kv_fp16=True)

"""From a model file to tokens on the GPU: the loaders (reference src/load_gguf.jl:317-394,
src/load_karpathy.jl:80-98) feed the device path, and text `sample` (src/inference.jl:317-395) drives it.

Each test writes a synthetic file with the package's own writer (the reference cannot write models and ships
none), loads it the way a user would, uploads the loaded arrays and compares the device's greedy tokens with the
oracle built from the same loaded arrays."""
import io
import re

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) / max(1e-30, np.max(np.abs(b))))


def _synthetic(pkg, plan, **kw):
    from llama2_jl_amd import synth
    return synth.synthetic_model(pkg.ModelConfig(**kw), getattr(synth, plan), seed=21,
                                 share_classifier=(plan == "PLAN_F32"))


def _check_against_oracle(pkg, orc, lm, n_new=32):
    from llama2_jl_amd import synth
    prompt = synth.seeded_prompt(3, 5, lm.config.vocab_size)
    dev = lm.device()
    om = orc.model_from_language_model(lm, nthreads=8)
    ids, logits = dev.generate_greedy(prompt, n_new, want_logits=True)
    ref_ids, ref_logits = om.generate_greedy(prompt, n_new, orc.GPU_SPEC)
    assert ids.tolist() == ref_ids.tolist()
    assert _rel(logits, ref_logits) <= 1e-3
    dev.close()
    om.close()


@pytest.mark.parametrize("mmap", [True, False])
def test_llama_gguf_file_to_tokens(pkg, orc, tmp_path, mmap):
    """llama architecture, Q4_K_S-style types with GQA: separate attn_q/k/v and ffn_gate/up tensors."""
    lm = _synthetic(pkg, "PLAN_Q4_K_S", dim=512, hidden_dim=1024, n_layers=2, n_heads=8, n_kv_heads=2, vocab_size=300,
                    seq_len=512, rope_freq_base=500000.0, rope_is_neox=False)
    path = str(tmp_path / "llama.gguf")
    pkg.save_gguf_model(path, lm, arch="llama")
    back = pkg.load_gguf_model(path, mmap=mmap)
    assert back.config.rope_is_neox is False and back.config.n_kv_heads == 2
    _check_against_oracle(pkg, orc, back)


def test_phi3_gguf_file_to_tokens(pkg, orc, tmp_path):
    """phi3 architecture: q, k, v are row ranges of one fused attn_qkv tensor and gate, up of one ffn_up tensor
    (src/load_gguf.jl:260-276): the loader hands out views of the mapped file, and those views are what is
    uploaded through l2h_model_set_tensor.  neox RoPE, no GQA."""
    from llama2_jl_amd.kquants import QuantMatrix
    lm = _synthetic(pkg, "PLAN_Q4_K", dim=512, hidden_dim=768, n_layers=2, n_heads=8, n_kv_heads=8, vocab_size=300,
                    seq_len=512, rope_freq_base=10000.0, rope_is_neox=True)
    path = str(tmp_path / "phi3.gguf")
    pkg.save_gguf_model(path, lm, arch="phi3")
    back = pkg.load_gguf_model(path, mmap=True)
    assert back.config.rope_is_neox is True
    l0 = back.weights.layers[0]
    assert isinstance(l0.wk, QuantMatrix) and (l0.wk.ne0, l0.wk.ne1) == (512, 512) and l0.w3.ne1 == 768
    assert np.array_equal(np.asarray(l0.wv.data), np.asarray(lm.weights.layers[0].wv.data))
    _check_against_oracle(pkg, orc, back)


def test_llama2c_file_to_tokens(pkg, orc, tmp_path):
    """llama2.c checkpoint + tokenizer.bin (src/load_karpathy.jl:1-98): fp32 weights, classifier shared with the
    embedding, hidden_dim not a multiple of 256."""
    lm = _synthetic(pkg, "PLAN_F32", dim=128, hidden_dim=344, n_layers=3, n_heads=4, n_kv_heads=4, vocab_size=260,
                    seq_len=96, rope_freq_base=10000.0, rope_is_neox=False)
    ckpt, tok = str(tmp_path / "model.bin"), str(tmp_path / "tokenizer.bin")
    pkg.save_karpathy_model(ckpt, tok, lm)
    back = pkg.load_karpathy_model(ckpt, tok)
    assert (back.config.dim, back.config.hidden_dim, back.config.seq_len) == (128, 344, 96)
    assert back.weights.output_weight is back.weights.token_embedding_table or \
        np.array_equal(back.weights.output_weight, back.weights.token_embedding_table)
    _check_against_oracle(pkg, orc, back)


def _toy_text_model(pkg):
    """a model whose vocabulary is a toy BPE table: single characters plus a few merges, so that encode() has
    merges to choose between by score (src/tokenizer.jl:29-54) and the printed text can be read back"""
    from llama2_jl_amd import synth
    from llama2_jl_amd.tokenizer import BPETokenizer
    pieces = [b"<unk>", b"<s>", b"</s>", b" "] + [bytes([c]) for c in b"abcdefghijklmnopqrstuvwxyz"] + \
        [b"th", b"he", b"the", b" the", b"an", b"and", b" a", b"in", b"er", b"on", b" o", b"re"]
    vocab = len(pieces)
    cfg = pkg.ModelConfig(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=vocab, seq_len=96,
                          rope_freq_base=10000.0, rope_is_neox=False)
    lm = synth.synthetic_model(cfg, synth.PLAN_Q4_K_S, seed=5)
    scores = [0.0] * 30 + [float(-i) for i in range(1, vocab - 30 + 1)]
    lm.tokenizer = BPETokenizer(pieces, scores, 1, 2)
    return lm


def test_text_sample_greedy_matches_generate(pkg):
    """sample() at temperature 0 (src/inference.jl:317-395): BOS in front of the encoded prompt (:338-340), tokens
    printed as they are chosen, the tok/s line at the end (:392).  What it prints is the text of the tokens that
    generate_greedy returns for the same token ids."""
    from llama2_jl_amd.tokenizer import encode, token_bytes
    lm = _toy_text_model(pkg)
    tok = lm.tokenizer
    prompt = "the cat and the hat"
    ids = [tok.bos_token_id] + encode(prompt, tok)
    assert len(ids) < 1 + len(prompt)  # some merge was taken
    n_total = 40
    out = io.StringIO()
    pkg.sample(lm, prompt, temperature=0.0, stop_on_special_token=False, max_seq_len=n_total, out=out)
    text = out.getvalue()
    m = re.search(r"\n-------\nachieved tok/s: (\d+\.\d\d)\n$", text)
    assert m and float(m.group(1)) > 0
    body = text[:m.start()]
    # the same steps on token ids: positions 0..n_total-1, of which the first len(ids)-1 only feed the prompt
    dev = lm.device()
    dev.reset()
    gen = dev.generate_greedy(ids, n_total - (len(ids) - 1))
    want = b"".join(token_bytes(tok, t) for t in ids[1:]) + b"".join(token_bytes(tok, int(t)) for t in gen)
    assert body == want.decode("utf-8", errors="replace")
    # with the stop rule: printing ends before the first BOS/EOS among the generated tokens (:371-373)
    out2 = io.StringIO()
    pkg.sample(lm, prompt, temperature=0.0, stop_on_special_token=True, max_seq_len=n_total, out=out2)
    body2 = out2.getvalue()[:out2.getvalue().index("\n-------")]
    special = [i for i, t in enumerate(gen) if int(t) in (tok.bos_token_id, tok.eos_token_id)]
    kept = gen[:special[0]] if special else gen
    want2 = b"".join(token_bytes(tok, t) for t in ids[1:]) + b"".join(token_bytes(tok, int(t)) for t in kept)
    assert body2 == want2.decode("utf-8", errors="replace")
    # bos_token=False prints the first prompt token itself (:342-344); an empty prompt is then an error (:326-328)
    out3 = io.StringIO()
    pkg.sample(lm, prompt, temperature=0.0, stop_on_special_token=False, max_seq_len=8, bos_token=False, out=out3)
    assert out3.getvalue().startswith(token_bytes(tok, encode(prompt, tok)[0]).decode())
    with pytest.raises(ValueError):
        pkg.sample(lm, "", bos_token=False, out=io.StringIO())


def test_text_sample_with_temperature(pkg):
    """temperature > 0 draws on the device (l2h_sample) with uniform numbers from the caller's generator: the same
    generator state gives the same text, and the text differs from the greedy one somewhere."""
    lm = _toy_text_model(pkg)
    outs = []
    for seed in (1, 1, 2):
        out = io.StringIO()
        pkg.sample(lm, "on the", temperature=1.5, stop_on_special_token=False, max_seq_len=48, rng=np.random.default_rng(seed),
                   out=out)
        outs.append(out.getvalue().split("\n-------")[0])
    g = io.StringIO()
    pkg.sample(lm, "on the", temperature=0.0, stop_on_special_token=False, max_seq_len=48, out=g)
    assert outs[0] == outs[1]
    assert outs[0] != outs[2] or outs[0] != g.getvalue().split("\n-------")[0]

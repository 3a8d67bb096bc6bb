"""Host-side logic that needs no GPU: the C-ABI library loads and exports every declared symbol,
the synthetic-weight factory and k-quant encoders, the GGUF and llama2.c loaders/writers with the
reference's accepted subset and error behaviour, and the tokenizers."""
import os
import re
import struct

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
Q4, Q5, Q6, F32 = 12, 13, 14, 0


def test_library_exports_every_declared_symbol(pkg):
    from llama2_jl_amd import _lib
    header = open(os.path.join(ROOT, "include", "l2h.h")).read()
    declared = set(re.findall(r"\b(l2h_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 30
    lib = _lib.lib()
    for name in declared:
        assert hasattr(lib, name), "libl2hip.so does not export " + name
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)


def _c_prototypes():
    """name -> list of C parameter types, from include/l2h.h"""
    header = open(os.path.join(ROOT, "include", "l2h.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    protos = {}
    for m in re.finditer(r"\b(?:int|void|const char \*)\s*\*?\s*(l2h_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", header, flags=re.S):
        params = [a.strip() for a in m.group(2).split(",")]
        protos[m.group(1)] = [] if params == ["void"] else params
    return protos


def _julia_class(t):
    """coarse class of a Julia ccall argument type"""
    t = t.strip()
    if t in ("Cint", "Int32", "UInt32", "Cuint"):
        return "i32"
    if t in ("Int64", "UInt64"):
        return "i64"
    if t in ("Cfloat", "Float32"):
        return "f32"
    if t.startswith("Ptr{") or t.startswith("Ref{") or t == "Cstring":
        return "ptr"
    raise AssertionError("unclassified Julia type " + t)


def _c_class(p):
    if "*" in p:
        return "ptr"
    base = " ".join(p.split()[:-1]) if len(p.split()) > 1 else p
    if base in ("int", "int32_t", "unsigned int", "uint32_t"):
        return "i32"
    if base in ("int64_t", "uint64_t"):
        return "i64"
    if base == "float":
        return "f32"
    raise AssertionError("unclassified C parameter " + p)


def test_julia_binding_matches_the_header():
    """Nobody can run Julia where this library is built, so the binding is checked as text: every ccall in
    llama2.jl_amd/julia/Llama2HIP.jl names a function the header declares, passes as many arguments as its
    prototype has, of the same class (32-bit integer, 64-bit integer, float, pointer) in the same order;
    and the functions the integration notes promise are defined at top level, outside any string."""
    src = open(os.path.join(ROOT, "llama2.jl_amd", "julia", "Llama2HIP.jl")).read()
    assert src.count('"""') % 2 == 0
    code = re.sub(r'""".*?"""', "", src, flags=re.S)      # docstrings out
    code = re.sub(r"(?m)#.*$", "", code)                   # comments out
    protos = _c_prototypes()
    assert len(protos) >= 30
    calls = list(re.finditer(r"ccall\(\(:(l2h_[a-z0-9_]+),\s*lib\),\s*(\w+),\s*\(([^()]*?)\),", code, flags=re.S))
    assert len(calls) >= 15
    for m in calls:
        name, ret, types = m.group(1), m.group(2), m.group(3)
        assert name in protos, name + " is not declared in include/l2h.h"
        jl = [t for t in (x.strip() for x in types.split(",")) if t]
        want = protos[name]
        assert len(jl) == len(want), "%s: %d ccall argument types, prototype has %d" % (name, len(jl), len(want))
        for i, (a, b) in enumerate(zip(jl, want)):
            assert _julia_class(a) == _c_class(b), "%s argument %d: Julia %s vs C %s" % (name, i, a, b)
        # the values passed: as many as the types (counted up to the call's closing parenthesis)
        depth, j = 1, m.end()
        args, cur = [], ""
        while depth > 0:
            ch = code[j]
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
                if depth == 0:
                    break
            if ch == "," and depth == 1:
                args.append(cur)
                cur = ""
            else:
                cur += ch
            j += 1
        args.append(cur)
        args = [a for a in (x.strip() for x in args) if a]
        assert len(args) == len(jl), "%s: %d values for %d argument types" % (name, len(args), len(jl))
        assert ret in ("Cint", "Cvoid", "Cstring")
    defined = set(re.findall(r"(?m)^function\s+([A-Za-z_!0-9]+)\s*\(", code)) | \
        set(re.findall(r"(?m)^([A-Za-z_!0-9]+)\([^\n]*\)\s*=", code))
    for fn in ("Context", "DeviceModel", "set_tensor!", "reset!", "transformer!", "generate", "prefill!", "sample_token",
               "sample", "matmul!", "dequantize!", "rmsnorm!", "rope!", "softmax!", "argmax_first", "kv_write!",
               "with_device_matrices", "on_device"):
        assert fn in defined, "Llama2HIP.%s is not defined" % fn
    # the drop-in seams: methods added to the reference's own generic functions, with the reference's argument lists
    # (src/matmul.jl:3-7, src/inference.jl:317-324), a matrix type for the AbstractMatrix fields of the weights
    # (src/inference.jl:27-48) and the resident-matrix product they rest on
    assert re.search(r"(?m)^function Llama2\.matmul!\(y::AbstractVector\{Float32\}, A::DeviceMatrix, x::AbstractVector\{Float32\}\)", code)
    assert re.search(r"(?m)^Llama2\.sample\(m::DeviceLanguageModel, prompt::String = \"\"; kwargs\.\.\.\)", code)
    assert re.search(r"(?m)^struct DeviceMatrix\{T, A <: AbstractMatrix\{T\}\} <: AbstractMatrix\{T\}", code)
    assert "l2h_model_matmul" in [m.group(1) for m in calls]


def test_no_device_is_an_error_not_a_fallback(pkg):
    """Without a GPU the context cannot be created; nothing computes on the CPU instead."""
    import ctypes
    from llama2_jl_amd import _lib
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    h = ctypes.c_void_p()
    rc = _lib.lib().l2h_ctx_create(0, ctypes.byref(h))
    assert rc in (_lib.ENODEV, _lib.EHIP) and not h.value
    assert len(_lib.lib().l2h_last_error(None)) > 0
    with pytest.raises(pkg.L2HError):
        pkg.Context(0)


def test_synth_normal_is_counter_based(pkg):
    from llama2_jl_amd import synth
    a = synth.normal(11, 3, (100000,), 0.02)
    assert abs(a.mean()) < 3e-4 and abs(a.std() - 0.02) < 3e-4
    assert abs(float(np.mean((a / 0.02) ** 4)) - 3.0) < 0.1  # kurtosis of a normal
    b = synth.normal(11, 3, (1000,), 0.02, offset=4321)  # any slice can be regenerated alone
    assert np.array_equal(b, a[4321:5321])
    assert not np.array_equal(synth.normal(11, 4, (1000,), 0.02), a[:1000])
    assert not np.array_equal(synth.normal(12, 3, (1000,), 0.02), a[:1000])


@pytest.mark.parametrize("typ,levels", [(Q4, 15), (Q5, 31), (Q6, 63)])
def test_weight_encoders_round_trip(pkg, orc, typ, levels):
    """Encoders emit valid blocks: decoding them with the reference's dequantize! (oracle) returns the
    input to within one quantization step of the sub-block's range."""
    from llama2_jl_amd import synth
    x = synth.normal(5, typ, (64, 1024), 0.02)
    x[0, :256] = 0  # an all-zero block
    x[1, :256] = np.abs(x[1, :256])  # no negative values: min clamps to 0
    q = pkg.quantize_weights(x, typ)
    assert q.data.size == 64 * 4 * {Q4: 144, Q5: 176, Q6: 210}[typ]
    y = orc.dequantize(typ, q.data).reshape(64, 1024)
    sub = 32 if typ != Q6 else 16
    xs, ys = x.reshape(-1, sub), y.reshape(-1, sub)
    rng_ = xs.max(1) - np.minimum(xs.min(1), 0) if typ != Q6 else 2 * np.abs(xs).max(1)
    err = np.abs(xs - ys).max(1)
    assert np.all(err <= 1.2 * rng_ / levels + 1e-7)
    assert np.all(y[0, :256] == 0)
    assert np.sqrt(np.mean((x - y) ** 2)) < {Q4: 0.0016, Q5: 0.0008, Q6: 0.0005}[typ]
    # threads only split the work
    x1 = np.ascontiguousarray(x)
    out1 = np.empty(q.data.size, np.uint8)
    from llama2_jl_amd import _lib
    assert _lib.lib().l2h_quantize_weights(typ, _lib.ptr(x1), x1.size, _lib.ptr(out1), 1) == 0
    assert np.array_equal(out1, q.data)
    assert _lib.lib().l2h_quantize_weights(typ, _lib.ptr(x1), 100, _lib.ptr(out1), 1) == _lib.EINVAL
    assert _lib.lib().l2h_quantize_weights(2, _lib.ptr(x1), 256, _lib.ptr(out1), 1) == _lib.ETYPE


def _tiny(pkg, plan="PLAN_Q4_K_S", **over):
    from llama2_jl_amd import synth
    kw = dict(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=40, seq_len=512,
              rope_freq_base=500000.0, rope_is_neox=False)
    kw.update(over)
    return synth.synthetic_model(pkg.ModelConfig(**kw), getattr(synth, plan), seed=3)


def _same_weights(a, b):
    from llama2_jl_amd.kquants import QuantMatrix
    def eq(x, y):
        if isinstance(x, QuantMatrix):
            return isinstance(y, QuantMatrix) and x.type == y.type and (x.ne0, x.ne1) == (y.ne0, y.ne1) and \
                np.array_equal(x.data, y.data)
        return np.array_equal(np.asarray(x), np.asarray(y))
    ok = eq(a.token_embedding_table, b.token_embedding_table) and eq(a.output_weight, b.output_weight) and \
        eq(a.rms_final_weight, b.rms_final_weight) and len(a.layers) == len(b.layers)
    for la, lb in zip(a.layers, b.layers):
        for f in ("rms_att_weight", "rms_ffn_weight", "wq", "wk", "wv", "wo", "w1", "w2", "w3"):
            ok = ok and eq(getattr(la, f), getattr(lb, f))
    return ok


@pytest.mark.parametrize("mmap", [True, False])
def test_gguf_round_trip_llama(pkg, tmp_path, mmap):
    lm = _tiny(pkg)
    path = str(tmp_path / "m.gguf")
    pkg.save_gguf_model(path, lm, arch="llama")
    back = pkg.load_gguf_model(path, mmap=mmap)
    assert back.config.seq_len == 512  # the reference hard-codes 512 (src/load_gguf.jl:237)
    assert back.config.rope_is_neox is False and abs(back.config.rope_freq_base - 500000.0) < 1
    assert (back.config.dim, back.config.hidden_dim, back.config.n_layers, back.config.n_heads,
            back.config.n_kv_heads, back.config.vocab_size) == (256, 512, 2, 4, 2, 40)
    assert _same_weights(lm.weights, back.weights)
    assert pkg.load_gguf_model(path, seq_len=4096).config.seq_len == 4096  # extension for long caches


def test_gguf_phi3_fused_tensors(pkg, tmp_path):
    """phi3 files fuse q,k,v and gate,up along the output rows (src/load_gguf.jl:260-276)."""
    lm = _tiny(pkg, "PLAN_Q4_K", n_kv_heads=4, rope_is_neox=True, rope_freq_base=10000.0)
    path = str(tmp_path / "p.gguf")
    pkg.save_gguf_model(path, lm, arch="phi3")
    meta, tensors = pkg.read_gguf(path)
    assert "blk.0.attn_qkv.weight" in tensors and "blk.0.attn_q.weight" not in tensors
    assert tensors["blk.0.attn_qkv.weight"].ne1 == 3 * 256 and tensors["blk.0.ffn_up.weight"].ne1 == 2 * 512
    back = pkg.load_gguf_model(path)
    assert back.config.rope_is_neox is True
    assert _same_weights(lm.weights, back.weights)


def test_gguf_errors(pkg, tmp_path):
    from llama2_jl_amd import gguf
    lm = _tiny(pkg)
    good = str(tmp_path / "g.gguf")
    pkg.save_gguf_model(good, lm)
    raw = bytearray(open(good, "rb").read())
    bad = str(tmp_path / "b.gguf")
    open(bad, "wb").write(b"GGML" + raw[4:])
    with pytest.raises(gguf.GGUFError, match="Not a GGUF file"):  # src/load_gguf.jl:87-89
        pkg.load_gguf_model(bad)
    # a metadata value of a type the reference cannot read (UINT64), src/load_gguf.jl:76
    head = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<IQ", gguf.T_UINT64, 5)
    open(bad, "wb").write(head)
    with pytest.raises(gguf.GGUFError, match="not implemented"):
        pkg.read_gguf(bad)
    # an F16 tensor (src/load_gguf.jl:153)
    gguf.write_gguf(bad, {"general.architecture": "llama"}, [])
    blob = open(bad, "rb").read()
    name = b"t.weight"
    info = struct.pack("<Q", len(name)) + name + struct.pack("<IQQIQ", 2, 256, 1, gguf.GGML_F16, 0)
    hdr = bytearray(blob)
    hdr[8:16] = struct.pack("<Q", 1)  # tensor_count = 1
    open(bad, "wb").write(bytes(hdr).rstrip(b"\0") + info + b"\0" * 1024)
    with pytest.raises(gguf.GGUFError, match="tensor type 1 not implemented"):
        pkg.read_gguf(bad)
    # ne0 not a multiple of 256 (src/load_gguf.jl:141)
    info = struct.pack("<Q", len(name)) + name + struct.pack("<IQQIQ", 2, 128, 2, gguf.GGML_Q4_K, 0)
    open(bad, "wb").write(bytes(hdr).rstrip(b"\0") + info + b"\0" * 1024)
    with pytest.raises(gguf.GGUFError, match="multiple of 256"):
        pkg.read_gguf(bad)
    # missing layer, unknown architecture, unknown tokenizer model (src/load_gguf.jl:213,370,389)
    meta, tensors = pkg.read_gguf(good)
    keep = [(k, v) for k, v in tensors.items() if not k.startswith("blk.1.")]
    plain = {k: v for k, v in meta.items() if k != "tokenizer.ggml.token_type"}
    typed = {"tokenizer.ggml.token_type": (gguf.T_ARRAY, list(meta["tokenizer.ggml.token_type"]))}
    gguf.write_gguf(bad, plain, keep, typed_meta=typed)
    with pytest.raises(gguf.GGUFError, match="missing blk.1 weights"):
        pkg.load_gguf_model(bad)
    gguf.write_gguf(bad, dict(plain, **{"general.architecture": "gpt-neox"}), list(tensors.items()), typed_meta=typed)
    with pytest.raises(gguf.GGUFError, match="unsupported model architecture"):
        pkg.load_gguf_model(bad)
    gguf.write_gguf(bad, dict(plain, **{"tokenizer.ggml.model": "bert"}), list(tensors.items()), typed_meta=typed)
    with pytest.raises(gguf.GGUFError, match="unsupported tokenizer model"):
        pkg.load_gguf_model(bad)
    open(bad, "wb").write(bytes(raw[:len(raw) // 2]))  # truncated
    with pytest.raises(gguf.GGUFError):
        pkg.load_gguf_model(bad)


def test_gguf_token_fixups(pkg, tmp_path):
    """llama tokenizer: the block character becomes a space in NORMAL tokens, <0xNN> BYTE tokens become
    the byte (src/load_gguf.jl:345-358); gpt2 tokenizer: byte-level unicode is undone (:359-368)."""
    from llama2_jl_amd import gguf
    lm = _tiny(pkg, vocab_size=6)
    tokens = ["<unk>", "<s>", "</s>", "▁the", "<0x0A>", "▁"]
    types = [2, 3, 3, 1, 6, 1]
    path = str(tmp_path / "t.gguf")
    pkg.save_gguf_model(path, lm, tokens=[t.encode() for t in tokens])
    meta, tensors = pkg.read_gguf(path)  # memory-mapped: write the variants to other files
    plain = {k: v for k, v in meta.items() if k != "tokenizer.ggml.token_type"}
    path2, path3 = str(tmp_path / "t2.gguf"), str(tmp_path / "t3.gguf")
    gguf.write_gguf(path2, plain, list(tensors.items()), typed_meta={"tokenizer.ggml.token_type": (gguf.T_ARRAY, types)})
    tok = pkg.load_gguf_model(path2).tokenizer
    assert tok.id_to_token == [b"<unk>", b"<s>", b"</s>", b" the", b"\n", b" "]
    assert (tok.bos_token_id, tok.eos_token_id) == (1, 2)
    dec = gguf.gpt2_decoder()
    assert len(dec) == 256 and sorted(dec.values()) == list(range(256))
    assert dec["Ġ"] == 32 and dec["A"] == 65 and dec["Ċ"] == 10  # 'Ġ' is space, 'Ċ' is newline
    gguf.write_gguf(path3, dict(plain, **{"tokenizer.ggml.model": "gpt2",
                                         "tokenizer.ggml.tokens": ["a", "b", "c", "Ġthe", "Ċ", "x"]}),
                    list(tensors.items()), typed_meta={"tokenizer.ggml.token_type": (gguf.T_ARRAY, [1] * 6)})
    assert pkg.load_gguf_model(path3).tokenizer.id_to_token[3:5] == [b" the", b"\n"]


def test_karpathy_round_trip(pkg, tmp_path):
    from llama2_jl_amd import synth
    cfg = pkg.ModelConfig(dim=64, hidden_dim=172, n_layers=2, n_heads=4, n_kv_heads=4, vocab_size=30, seq_len=32)
    lm = synth.synthetic_model(cfg, synth.PLAN_F32, seed=9, share_classifier=True)
    ck, tk = str(tmp_path / "m.bin"), str(tmp_path / "tok.bin")
    pkg.save_karpathy_model(ck, tk, lm)
    assert os.path.getsize(ck) == 28 + 4 * (30 * 64 + 2 * (64 + 4 * 64 * 64 + 64 + 3 * 172 * 64) + 64)
    back = pkg.load_karpathy_model(ck, tk)
    c = back.config
    assert (c.dim, c.hidden_dim, c.n_layers, c.n_heads, c.n_kv_heads, c.vocab_size, c.seq_len) == (64, 172, 2, 4, 4, 30, 32)
    assert c.rope_freq_base == 10000.0 and c.rope_is_neox is False  # src/load_karpathy.jl:9-10
    assert _same_weights(lm.weights, back.weights)
    assert back.weights.output_weight is back.weights.token_embedding_table  # shared classifier (:56)
    assert back.tokenizer.id_to_token == lm.tokenizer.id_to_token
    assert (back.tokenizer.bos_token_id, back.tokenizer.eos_token_id) == (1, 2)  # the reference's 2, 3 one-based
    open(ck, "ab").write(b"\0" * 64)  # trailing bytes (legacy freq_cis) are ignored
    assert _same_weights(lm.weights, pkg.load_karpathy_model(ck, tk).weights)
    data = open(ck, "rb").read()
    open(ck, "wb").write(data[:len(data) // 2])
    with pytest.raises(ValueError, match="truncated"):
        pkg.load_karpathy_model(ck, tk)
    open(ck, "wb").write(data[:10])
    with pytest.raises(ValueError, match="header"):
        pkg.load_karpathy_model(ck, tk)


def test_bpe_encode(pkg):
    """encode() (src/tokenizer.jl:11-57): one token per byte, then the best-scoring adjacent pair is
    merged until none is left; a leading space token is added first."""
    toks = [b"<unk>", b"<s>", b"</s>", b" ", b"a", b"b", b"c", b"ab", b"bc", b"abc", b" a", b" ab"]
    scores = [0, 0, 0, 0, 0, 0, 0, 1.0, 2.0, 3.0, 0.5, 4.0]
    t = pkg.BPETokenizer(toks, scores, 1, 2)
    assert pkg.encode("", t) == []
    # " abc": bytes [' ', a, b, c]; candidates " a"(.5), "ab"(1), "bc"(2) -> "bc" first; then " a"(.5) only
    # (a + "bc" = "abc" scores 3 and beats it) -> "abc"; then " " + "abc" is no token: done
    assert [toks[i] for i in pkg.encode("abc", t)] == [b" ", b"abc"]
    assert [toks[i] for i in pkg.encode("ab", t)] == [b" ab"]  # "ab"(1) first, then " "+"ab" = " ab"(4)
    assert [toks[i] for i in pkg.encode("abc", t, pad_input=False)] == [b"abc"]
    assert [toks[i] for i in pkg.encode("cab", t, pad_input=False)] == [b"c", b"ab"]
    assert t.decode(pkg.encode("abc", t)) == " abc"
    with pytest.raises(KeyError):
        pkg.encode("z", t)  # a byte without a token, as token_to_id[...] throws in the reference


def test_char_tokenizer(pkg):
    t = pkg.CharTokenizer("hello world")  # src/tokenizer.jl:59-80
    assert t.id_to_token == [" ", "d", "e", "h", "l", "o", "r", "w", "<s>", "</s>"]
    assert (t.bos_token_id, t.eos_token_id) == (8, 9)
    assert pkg.encode("low", t) == [4, 5, 7]
    assert t.decode([3, 2, 4, 4, 5]) == "hello"


def test_quant_matrix_views(pkg, rng):
    raw = rng.integers(0, 256, 6 * 2 * 144, dtype=np.uint8)
    A = pkg.QuantMatrix(Q4, raw, 512, 6)
    assert A.shape == (512, 6) and A.blocks.shape == (6, 2)
    v = A.rows(2, 5)
    assert (v.ne0, v.ne1) == (512, 3) and np.array_equal(v.data, raw[2 * 288:5 * 288])
    with pytest.raises(ValueError):
        pkg.QuantMatrix(Q4, raw, 500, 6)
    with pytest.raises(ValueError):
        pkg.QuantMatrix(2, raw, 512, 6)
    with pytest.raises(ValueError):
        pkg.QuantMatrix(Q4, raw[:-1], 512, 6)


def test_weight_bytes_match_the_published_table(pkg):
    """Bytes streamed per token at the headline shape: 4.3568 GB (q4_K layers + q6_K classifier)."""
    per_layer = (4096 * 4096 * 2 + 4096 * 1024 * 2 + 3 * 4096 * 14336) // 256 * 144
    assert per_layer == 122683392
    assert 32 * per_layer + 4096 * 128256 // 256 * 210 == 4356808704

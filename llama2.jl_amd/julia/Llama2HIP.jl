# Llama2HIP.jl -- Julia binding of libl2hip.so for Llama2.jl users.
#
# Keeps the package surface of Llama2.jl (load_gguf_model, load_karpathy_model, LanguageModel,
# sample): the loaders and tokenizers are Llama2.jl's own; only the per-token forward pass and the
# greedy loop run on the GPU through `ccall`.  Token ids and positions are 1-based on this side and
# 0-based in the C ABI (include/l2h.h).
#
# NOT EXERCISED BY THE TEST SUITE: no Julia toolchain is available where this library is built and
# tested; the Python binding (llama2.jl_amd/_lib.py) calls the same symbols and is the tested one.
module Llama2HIP

using Llama2
import Llama2
using Llama2: LanguageModel, ModelConfig, TransformerWeights, TransformerLayerWeights,
              block_q4_K, block_q5_K, block_q6_K, encode

const lib = get(ENV, "L2H_LIB", joinpath(@__DIR__, "..", "libl2hip.so"))

struct L2HConfig            # l2h_config
    dim::Int32; hidden_dim::Int32; n_layers::Int32; n_heads::Int32; n_kv_heads::Int32
    vocab_size::Int32; seq_len::Int32; rope_freq_base::Float32; rope_is_neox::Int32
end

# tensor roles and GGML types of include/l2h.h
const TOK_EMB, RMS_FINAL, OUTPUT, RMS_ATT, RMS_FFN, WQ, WK, WV, WO, W1, W2, W3 = 0:11
ggml_type(::AbstractArray{Float32}) = 0
ggml_type(::AbstractArray{block_q4_K}) = 12
ggml_type(::AbstractArray{block_q5_K}) = 13
ggml_type(::AbstractArray{block_q6_K}) = 14

mutable struct Context
    handle::Ptr{Cvoid}
end

function check(ctx::Ptr{Cvoid}, rc::Cint)
    rc == 0 && return
    msg = unsafe_string(ccall((:l2h_last_error, lib), Cstring, (Ptr{Cvoid},), ctx))
    error("l2h error $rc: $msg")
end

function Context(device::Integer = 0)
    h = Ref{Ptr{Cvoid}}(C_NULL)
    rc = ccall((:l2h_ctx_create, lib), Cint, (Cint, Ref{Ptr{Cvoid}}), device, h)
    check(Ptr{Cvoid}(C_NULL), rc)
    ctx = Context(h[])
    finalizer(c -> ccall((:l2h_ctx_destroy, lib), Cvoid, (Ptr{Cvoid},), c.handle), ctx)
    return ctx
end

mutable struct DeviceModel
    ctx::Context
    handle::Ptr{Cvoid}
    config::ModelConfig
end

# (in_features, out_rows) of a weight as matmul! sees it; k-quant arrays hold in/256 blocks per row
in_out(A::AbstractMatrix{Float32}) = size(A)
in_out(A::AbstractMatrix) = (size(A, 1) * 256, size(A, 2))
in_out(v::AbstractVector{Float32}) = (length(v), 1)

function set_tensor!(m::DeviceModel, role, layer, A)
    host = A isa Array ? A : collect(A)          # views (Phi-3 fused tensors) and mmaps become dense
    ne0, ne1 = in_out(host)
    GC.@preserve host begin
        rc = ccall((:l2h_model_set_tensor, lib), Cint,
                   (Ptr{Cvoid}, Cint, Cint, Cint, Ptr{Cvoid}, Int64, Int64),
                   m.handle, role, layer, ggml_type(host), pointer(host), ne0, ne1)
    end
    check(m.ctx.handle, rc)
end

"""
Upload the weights of a Llama2.jl `LanguageModel` once; the copy stays resident in HBM.  `kv_fp16 = true` keeps
the KV cache in Float16 (rows rounded when appended; the reference's cache is Float32, `src/inference.jl:62-70`).
"""
function DeviceModel(model::LanguageModel; ctx::Context = Context(), seq_len::Integer = model.config.seq_len,
                     kv_fp16::Bool = false)
    c = model.config
    cfg = L2HConfig(c.dim, c.hidden_dim, c.n_layers, c.n_heads, c.n_kv_heads, c.vocab_size, seq_len,
                    c.rope_freq_base, c.rope_is_neox ? 1 : 0)
    h = Ref{Ptr{Cvoid}}(C_NULL)
    check(ctx.handle, ccall((:l2h_model_create, lib), Cint, (Ptr{Cvoid}, Ref{L2HConfig}, Ref{Ptr{Cvoid}}),
                            ctx.handle, cfg, h))
    m = DeviceModel(ctx, h[], c)
    finalizer(x -> ccall((:l2h_model_destroy, lib), Cvoid, (Ptr{Cvoid},), x.handle), m)
    w = model.weights
    set_tensor!(m, TOK_EMB, 0, w.token_embedding_table)
    set_tensor!(m, RMS_FINAL, 0, w.rms_final_weight)
    set_tensor!(m, OUTPUT, 0, w.output_weight)
    for (l, lw) in enumerate(w.layers)
        for (role, A) in ((RMS_ATT, lw.rms_att_weight), (RMS_FFN, lw.rms_ffn_weight), (WQ, lw.wq), (WK, lw.wk),
                          (WV, lw.wv), (WO, lw.wo), (W1, lw.w1), (W2, lw.w2), (W3, lw.w3))
            set_tensor!(m, role, l - 1, A)
        end
    end
    kv_fp16 && check(ctx.handle, ccall((:l2h_model_set_kv_type, lib), Cint, (Ptr{Cvoid}, Cint), m.handle, 1))
    check(ctx.handle, ccall((:l2h_model_finalize, lib), Cint, (Ptr{Cvoid},), m.handle))
    return m
end

"Which of the library's launch paths decodes this model (3 = the one-launch-per-token streaming kernel), and why not 3."
launch_path(m::DeviceModel) = Int(ccall((:l2h_model_path, lib), Cint, (Ptr{Cvoid},), m.handle))
launch_path_reason(m::DeviceModel) = unsafe_string(ccall((:l2h_model_path_reason, lib), Cstring, (Ptr{Cvoid},), m.handle))
"Steps of the token loop (src/inference.jl:349-386) that one kernel launch of `generate` runs."
steps_per_launch(m::DeviceModel) = Int(ccall((:l2h_model_steps_per_launch, lib), Cint, (Ptr{Cvoid},), m.handle))
"Whether `prefill!` runs its plain products (q|k|v, wo, w2) through hipBLASLt (default) or through the library's own kernels."
set_prefill_library!(m::DeviceModel, on::Bool) =
    check(m.ctx.handle, ccall((:l2h_model_set_prefill_library, lib), Cint, (Ptr{Cvoid}, Cint), m.handle, on ? 1 : 0))
prefill_library(m::DeviceModel) = ccall((:l2h_model_prefill_library, lib), Cint, (Ptr{Cvoid},), m.handle) != 0

reset!(m::DeviceModel) = check(m.ctx.handle, ccall((:l2h_state_reset, lib), Cint, (Ptr{Cvoid},), m.handle))

"transformer!(token, pos, ...) of Llama2.jl (src/inference.jl:222): fills `logits`, returns argmax (1-based)."
function transformer!(logits::Vector{Float32}, m::DeviceModel, token::Int, pos::Int)
    am = Ref{Int32}(0)
    check(m.ctx.handle, ccall((:l2h_forward, lib), Cint, (Ptr{Cvoid}, Cint, Cint, Ptr{Float32}, Ref{Int32}),
                              m.handle, token - 1, pos - 1, logits, am))
    return Int(am[]) + 1
end

"Greedy continuation of 1-based token ids entirely on the device (the loop of sample() at temperature 0)."
function generate(m::DeviceModel, prompt::Vector{Int}, n_new::Int; pos::Int = 1)
    p = Int32.(prompt .- 1)
    out = Vector{Int32}(undef, n_new)
    check(m.ctx.handle, ccall((:l2h_generate_greedy, lib), Cint,
                              (Ptr{Cvoid}, Ptr{Int32}, Cint, Cint, Cint, Ptr{Int32}, Ptr{Float32}),
                              m.handle, p, length(p), pos - 1, n_new, out, C_NULL))
    return Int.(out) .+ 1
end

# Whole prompt in one pass on the matrix cores (no counterpart in Llama2.jl, which feeds the prompt token
# by token): fills the cache for positions pos .. pos+length(prompt)-1 and returns the next token (1-based).
function prefill!(m::DeviceModel, prompt::Vector{Int}; pos::Int = 1)
    p0 = Int32.(prompt .- 1)
    next = Ref{Int32}(0)
    check(m.ctx.handle, ccall((:l2h_prefill, lib), Cint,
                              (Ptr{Cvoid}, Ptr{Int32}, Cint, Cint, Ptr{Float32}, Ref{Int32}),
                              m.handle, p0, length(p0), pos - 1, C_NULL, next))
    return Int(next[]) + 1
end

# Temperature branch of sample (src/inference.jl:363-367) on the logits the last step left on the device;
# u stands in for wsample's draw from the global RNG.
function sample_token(m::DeviceModel, temperature::Float32; u::Float32 = min(rand(Float32), prevfloat(1f0)))
    tok = Ref{Int32}(0)
    check(m.ctx.handle, ccall((:l2h_sample, lib), Cint, (Ptr{Cvoid}, Cfloat, Cfloat, Ref{Int32}, Ptr{Float32}),
                              m.handle, temperature, u, tok, C_NULL))
    return Int(tok[]) + 1
end

# One step without copying the logits back: returns the argmax (1-based); the logits stay on the device
# for sample_token.
function step!(m::DeviceModel, token::Int, pos::Int)
    am = Ref{Int32}(0)
    check(m.ctx.handle, ccall((:l2h_forward, lib), Cint, (Ptr{Cvoid}, Cint, Cint, Ptr{Float32}, Ref{Int32}),
                              m.handle, token - 1, pos - 1, C_NULL, am))
    return Int(am[]) + 1
end

"""
    sample(m::DeviceModel, model::LanguageModel, prompt=""; temperature=0.9f0, stop_on_special_token=true,
           max_seq_len=typemax(Int), bos_token=true)

Same behaviour and output as `Llama2.sample` (src/inference.jl:317-395): the prompt is encoded with the
model's tokenizer, BOS is pushed in front (:338-340), tokens are printed as they are chosen, generation
stops at BOS/EOS (:371-373) and the tok/s line closes the output (:392).  The forward pass, the argmax
and the temperature draw run on the device; the uniform number of the draw comes from Julia's RNG.
"""
function sample(m::DeviceModel, model::LanguageModel, prompt::String = ""; temperature::Float32 = 0.9f0,
                stop_on_special_token = true, max_seq_len = typemax(Int), bos_token = true)
    !bos_token && isempty(prompt) && error("Prompt cannot be empty if bos_token = false")
    config, tokenizer = model.config, model.tokenizer
    prompt_tokens = encode(prompt, tokenizer)
    reset!(m)
    time_start = time_ns()
    bos_token && pushfirst!(prompt_tokens, tokenizer.bos_token_id)
    !bos_token && print(tokenizer.id_to_token[prompt_tokens[1]])
    token = prompt_tokens[1]
    generated_seq_len = 0
    for pos in 1:min(config.seq_len, max_seq_len)
        am = step!(m, token, pos)
        generated_seq_len += 1
        if pos + 1 <= length(prompt_tokens)
            next = prompt_tokens[pos + 1]
        elseif temperature == 0f0
            next = am
        else
            next = sample_token(m, temperature)
        end
        if stop_on_special_token && (next == tokenizer.bos_token_id || next == tokenizer.eos_token_id)
            break
        end
        print(tokenizer.id_to_token[next])
        token = next
    end
    println()
    println("-------\nachieved tok/s: ", round(generated_seq_len / (time_ns() - time_start) * 1e9; digits = 2))
    return nothing
end

# ---- drop-in use: the package's own entry points on device-resident weights ------------------------------------
#
# Two seams, both without a changed line in Llama2.jl:
#
#  * `DeviceLanguageModel` is a model type of its own for which `Llama2.sample` has a method, so that
#        model = on_device(load_gguf_model("model.gguf"));  sample(model, "Once upon a time")
#    reads like the reference's call (src/inference.jl:317-324) and runs the whole token loop on the GPU.
#  * `DeviceMatrix <: AbstractMatrix` stands in for a weight in the `AbstractMatrix` fields of
#    `TransformerWeights` / `TransformerLayerWeights` (src/inference.jl:27-48).  `Llama2.matmul!` has a method for it
#    (the reference dispatches on the matrix type, src/matmul.jl:3-23), so a `LanguageModel` built by
#    `with_device_matrices` flows through the reference's own `sample` and `transformer!` unchanged: rmsnorm, RoPE and
#    attention stay on the CPU, every matrix product runs on the resident weights (one vector up, one down per product:
#    the slow of the two seams, for checking one against the other).

"A weight that lives in a `DeviceModel`: `matmul!` runs on the GPU, everything else (size, indexing) on the host array."
struct DeviceMatrix{T, A <: AbstractMatrix{T}} <: AbstractMatrix{T}
    dev::DeviceModel
    role::Int32
    layer::Int32          # 0-based, as the C ABI counts
    host::A
end
Base.size(A::DeviceMatrix) = size(A.host)
Base.getindex(A::DeviceMatrix, i::Int, j::Int) = A.host[i, j]
Base.getindex(A::DeviceMatrix, ::Colon, j::Int) = A.host[:, j]
Base.view(A::DeviceMatrix, ::Colon, j::Int) = view(A.host, :, j)
Base.IndexStyle(::Type{<:DeviceMatrix}) = IndexCartesian()

"`matmul!(y, A, x)` of Llama2.jl (src/matmul.jl:3-23) for a device-resident `A`."
function Llama2.matmul!(y::AbstractVector{Float32}, A::DeviceMatrix, x::AbstractVector{Float32})
    xs = x isa Vector{Float32} ? x : collect(x)
    ys = y isa Vector{Float32} ? y : Vector{Float32}(undef, length(y))
    check(A.dev.ctx.handle, ccall((:l2h_model_matmul, lib), Cint, (Ptr{Cvoid}, Cint, Cint, Ptr{Float32}, Ptr{Float32}),
                                  A.dev.handle, A.role, A.layer, xs, ys))
    ys === y || copyto!(y, ys)
    return nothing
end

"A `LanguageModel` whose matrices are `DeviceMatrix`es of `dev`: the reference's `sample(model, prompt)` runs on it as it is."
function with_device_matrices(model::LanguageModel, dev::DeviceModel = DeviceModel(model))
    w = model.weights
    dm(role, layer, A) = DeviceMatrix{eltype(A), typeof(A)}(dev, Int32(role), Int32(layer), A)
    layers = [TransformerLayerWeights(; rms_att_weight = lw.rms_att_weight, rms_ffn_weight = lw.rms_ffn_weight,
                                      wq = dm(WQ, l - 1, lw.wq), wk = dm(WK, l - 1, lw.wk), wv = dm(WV, l - 1, lw.wv),
                                      wo = dm(WO, l - 1, lw.wo), w1 = dm(W1, l - 1, lw.w1), w2 = dm(W2, l - 1, lw.w2),
                                      w3 = dm(W3, l - 1, lw.w3)) for (l, lw) in enumerate(w.layers)]
    weights = TransformerWeights(; token_embedding_table = w.token_embedding_table, layers = layers,
                                 rms_final_weight = w.rms_final_weight, output_weight = dm(OUTPUT, 0, w.output_weight))
    return LanguageModel(model.config, model.tokenizer, weights)
end

"A loaded model together with its resident copy: what `sample` takes in place of a `LanguageModel`."
struct DeviceLanguageModel{TOK}
    host::LanguageModel{TOK}
    dev::DeviceModel
end
on_device(model::LanguageModel; kwargs...) = DeviceLanguageModel(model, DeviceModel(model; kwargs...))
# (config, tokenizer and weights read as on a LanguageModel)
Base.getproperty(m::DeviceLanguageModel, name::Symbol) =
    name === :host || name === :dev ? getfield(m, name) : getproperty(getfield(m, :host), name)

"`sample(model, prompt; ...)` of Llama2.jl (src/inference.jl:317-395), the token loop on the GPU."
Llama2.sample(m::DeviceLanguageModel, prompt::String = ""; kwargs...) = sample(m.dev, m.host, prompt; kwargs...)

# ---- the single operators (each one seam of src/inference.jl / src/matmul.jl; host arrays in, host arrays out) ----

"`matmul!(y, A, x)` (src/matmul.jl:3-23) on the GPU: A is `(in, out)` of Float32 or `(in ÷ 256, out)` of k-quant blocks."
function matmul!(ctx::Context, y::Vector{Float32}, A::AbstractMatrix, x::Vector{Float32})
    host = A isa Array ? A : collect(A)
    ne0, ne1 = in_out(host)
    @assert length(x) == ne0 && length(y) == ne1
    GC.@preserve host check(ctx.handle, ccall((:l2h_matmul, lib), Cint,
        (Ptr{Cvoid}, Cint, Ptr{Cvoid}, Int64, Int64, Ptr{Float32}, Ptr{Float32}, Ptr{Int32}, Ptr{Int32}),
        ctx.handle, ggml_type(host), pointer(host), ne0, ne1, x, y, C_NULL, C_NULL))
    return y
end

"`dequantize!(y, x)` (src/kquants.jl:70-125, 186-251, 322-363) of a vector of k-quant blocks."
function dequantize!(ctx::Context, y::Vector{Float32}, x::Vector{T}) where {T <: Union{block_q4_K, block_q5_K, block_q6_K}}
    @assert length(y) == 256 * length(x)
    check(ctx.handle, ccall((:l2h_dequantize, lib), Cint, (Ptr{Cvoid}, Cint, Ptr{Cvoid}, Int64, Ptr{Float32}),
                            ctx.handle, ggml_type(x), x, length(x), y))
    return y
end

"`rmsnorm!(o, x, weight)` (src/inference.jl:102-110); `o` may be `x`."
function rmsnorm!(ctx::Context, o::Vector{Float32}, x::Vector{Float32}, weight::Vector{Float32})
    check(ctx.handle, ccall((:l2h_rmsnorm, lib), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}, Int64),
                            ctx.handle, o, x, weight, length(x)))
    return o
end

"`rope!(x, pos, config)` (src/inference.jl:112-167) on `x` of `(head_size, n_heads)`; `pos` is 1-based."
function rope!(ctx::Context, x::Matrix{Float32}, pos::Int, config::ModelConfig)
    check(ctx.handle, ccall((:l2h_rope, lib), Cint, (Ptr{Cvoid}, Ptr{Float32}, Cint, Cint, Cint, Cfloat, Cint),
                            ctx.handle, x, size(x, 1), size(x, 2), pos - 1, config.rope_freq_base, config.rope_is_neox ? 1 : 0))
    return x
end

"`softmax!(x)` (src/inference.jl:169-174)."
function softmax!(ctx::Context, x::Vector{Float32})
    check(ctx.handle, ccall((:l2h_softmax, lib), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64), ctx.handle, x, length(x)))
    return x
end

"First index of the largest element, 1-based, as `argmax(logits)` in `sample` (src/inference.jl:360)."
function argmax_first(ctx::Context, x::Vector{Float32})
    out = Ref{Int32}(0)
    check(ctx.handle, ccall((:l2h_argmax, lib), Cint, (Ptr{Cvoid}, Ptr{Float32}, Int64, Ref{Int32}), ctx.handle, x, length(x), out))
    return Int(out[]) + 1
end

"Rows `pos .. pos+n-1` (1-based) of a layer's K and V cache, each `(kv_dim, n)` on this side (src/inference.jl:259-260)."
function kv_write!(m::DeviceModel, layer::Int, pos::Int, k::Matrix{Float32}, v::Matrix{Float32})
    @assert size(k) == size(v)
    check(m.ctx.handle, ccall((:l2h_kv_write, lib), Cint, (Ptr{Cvoid}, Cint, Cint, Cint, Ptr{Float32}, Ptr{Float32}),
                              m.handle, layer - 1, pos - 1, size(k, 2), k, v))
end

end # module

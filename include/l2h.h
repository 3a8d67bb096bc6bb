/*
 * l2h.h -- C ABI of libl2hip.so: Llama2.jl's per-token decode path on one MI355X (gfx950).
 *
 * The reference (cafaxo/Llama2.jl) is pure Julia and has no FFI layer; its seams are
 * Julia generic functions.  Each entry point below names the Julia function or type it
 * stands in for (paths relative to the Llama2.jl source tree).  A Julia `ccall`, a Python
 * `ctypes` or a C caller binds the same symbols.
 *
 * Conventions
 *   - every function returns 0 on success or a negative L2H_E* code; the message of the
 *     last failure on a context is l2h_last_error(ctx) (thread-unsafe, like the handles);
 *   - token ids and positions are 0-based here (Julia callers subtract 1);
 *   - host pointers passed in are borrowed for the duration of the call only;
 *   - handles are opaque and owned by the library; one host thread per context;
 *   - weights are uploaded once by l2h_model_set_tensor and stay resident in HBM in the
 *     library's own layout; the KV cache and all activations live in HBM.
 */
#ifndef L2H_H
#define L2H_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct l2h_ctx l2h_ctx;
typedef struct l2h_model l2h_model;

enum {
    L2H_OK = 0,
    L2H_EINVAL = -1,   /* bad argument (shape, role, range) */
    L2H_ETYPE = -2,    /* tensor type not one of F32/Q4_K/Q5_K/Q6_K (load_gguf.jl:153) */
    L2H_ESTATE = -3,   /* call out of order (e.g. forward before finalize) */
    L2H_EHIP = -4,     /* a HIP runtime call failed */
    L2H_ENOMEM = -5,
    L2H_ENODEV = -6    /* no usable gfx950 device */
};

/* GGML tensor types accepted, numbered as in GGUF (src/load_gguf.jl:26-42). */
enum { L2H_TYPE_F32 = 0, L2H_TYPE_Q4_K = 12, L2H_TYPE_Q5_K = 13, L2H_TYPE_Q6_K = 14 };

/* Tensor roles: the fields of TransformerWeights / TransformerLayerWeights
 * (src/inference.jl:27-48). */
enum {
    L2H_TOK_EMB = 0,   /* token_embedding_table (dim, vocab)      */
    L2H_RMS_FINAL = 1, /* rms_final_weight (dim,) F32             */
    L2H_OUTPUT = 2,    /* output_weight (dim, vocab)              */
    L2H_RMS_ATT = 3,   /* rms_att_weight (dim,) F32               */
    L2H_RMS_FFN = 4,   /* rms_ffn_weight (dim,) F32               */
    L2H_WQ = 5,        /* wq (dim, dim)                           */
    L2H_WK = 6,        /* wk (dim, kv_dim)                        */
    L2H_WV = 7,        /* wv (dim, kv_dim)                        */
    L2H_WO = 8,        /* wo (dim, dim)                           */
    L2H_W1 = 9,        /* w1 (dim, hidden)   ffn_gate             */
    L2H_W2 = 10,       /* w2 (hidden, dim)   ffn_down             */
    L2H_W3 = 11,       /* w3 (dim, hidden)   ffn_up               */
    L2H_N_ROLES = 12
};

/* ModelConfig (src/inference.jl:1-11). */
typedef struct l2h_config {
    int32_t dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len;
    float rope_freq_base;
    int32_t rope_is_neox;
} l2h_config;

/* ---- context ----------------------------------------------------------------------- */
/* Binds a HIP device and creates the stream all work of this context runs on. */
int l2h_ctx_create(int device, l2h_ctx **out);
void l2h_ctx_destroy(l2h_ctx *ctx);
const char *l2h_last_error(l2h_ctx *ctx); /* ctx may be NULL: error of a failed ctx_create */
int l2h_sync(l2h_ctx *ctx);
/* name of the device, compute units, HBM bytes; any pointer may be NULL */
int l2h_device_info(l2h_ctx *ctx, char *name, int name_cap, int32_t *n_cu, int64_t *hbm_bytes);

/* ---- model: TransformerWeights + RunState (src/inference.jl:27-100) ----------------- */
int l2h_model_create(l2h_ctx *ctx, const l2h_config *cfg, l2h_model **out);
void l2h_model_destroy(l2h_model *m);
/* Stands in for storing a host array in a TransformerWeights field: `host` holds ne1
 * output rows of ne0 input features, row-contiguous, as GGUF stores them and as
 * `view(A, :, i)` hands them to vecdot (src/matmul.jl:19).  k-quant types need
 * ne0 % 256 == 0 (src/load_gguf.jl:141) and ne0 <= 16384 (the longest activation vector the
 * matvec kernels stage; L2H_EINVAL beyond it).  Repacks into the device layout and uploads.
 * layer is ignored for the three per-model roles. */
int l2h_model_set_tensor(l2h_model *m, int role, int layer, int ggml_type, const void *host, int64_t ne0,
                         int64_t ne1);
/* Reads a k-quant tensor back from the device layout into GGUF block order (the repack
 * is exactly invertible); host must hold ne1 * ne0/256 blocks.  For checks. */
int l2h_model_get_tensor(l2h_model *m, int role, int layer, void *host, int64_t host_bytes);
/* Element type of the KV cache (before finalize).  L2H_KV_F32, the default, is the reference's KVCache
 * (Float32 arrays, src/inference.jl:62-70) and the parity path.  L2H_KV_F16 has no counterpart in the
 * reference: the rows appended by transformer! (and those passed to l2h_kv_write) are rounded to binary16
 * (nearest even) and widened again when the attention reads them, so a decode step reads half the cache
 * bytes; everything else computes as before.  Needs a head size that is a multiple of 32, at most 128; runs
 * on launch paths 1 and 3 (not 2); l2h_prefill is not available (L2H_ESTATE).  l2h_kv_read returns the
 * rounded values. */
enum { L2H_KV_F32 = 0, L2H_KV_F16 = 1 };
int l2h_model_set_kv_type(l2h_model *m, int kv_type);
/* How transformer! is launched (before finalize): 0 = automatic (3 where the model fits it, else 1),
 * 1 = one kernel per phase (recorded once, replayed per token), 2 = a persistent kernel per token
 * with grid barriers between the phases, 3 = the streaming kernel per token (per-wavefront weight
 * streams fetched ahead into LDS, activations exchanged as epoch-tagged words).  Path 3 takes
 *   - q4_K, q5_K or q6_K layer matrices (w1 and w3 of a layer of one type) with a q4_K or q6_K classifier:
 *     dim a multiple of 256, at most 4096, and either a multiple of 2048 or at most a quarter below one
 *     (1536..2048, 3072..4096; a q6_K classifier needs the multiple of 2048 above dim to be 4096);
 *     hidden_dim a multiple of 2048 up to 14336; head size 32, 64, 96 or 128; fp32 or fp16 cache;
 *   - models whose matrices are all fp32: dim and hidden_dim multiples of 4, at most 4096; head size 32, 64
 *     or 128; fp32 cache;
 *   in both cases n_heads <= 256, a head size that is a multiple of 256 / n_heads, and a cache length that fits
 *   the attention's LDS area (with head size 128: about 2 400 positions times 256 / n_heads, e.g. 19 000
 *   for 32 heads).
 * 2 and 3 are an error at finalize if the model does not fit; l2h_model_path_reason then tells why.  All paths compute the same
 * arithmetic and give the same results.  No counterpart in the reference.  l2h_model_path reports
 * the choice after finalize (1, 2 or 3). */
int l2h_model_set_path(l2h_model *m, int path);
int l2h_model_path(l2h_model *m);
/* Steps of the token loop (src/inference.jl:349-386) that one kernel launch of l2h_generate_greedy runs: 1, or up to 8
 * on path 3 for a model in which no two heads share a cache row (n_kv_heads == n_heads; the cache then lies in uncached
 * memory).  No counterpart in the reference. */
int l2h_model_steps_per_launch(l2h_model *m);
/* After finalize with the automatic choice: why the streaming kernel (path 3) was not taken, e.g. "layer matrices
 * must be q4_K" for a file whose first layers hold q5_K attn_v / ffn_down tensors; "" when it was taken.  The
 * string lives as long as the model. */
const char *l2h_model_path_reason(l2h_model *m);
/* Launch paths 2 and 3 wait on the device for other workgroups' results; every such wait gives up after
 * `spins` polls (default 2^20 on path 3, about a second), upon which all workgroups leave the kernel and
 * the call that launched it returns L2H_EHIP; the model stays usable (l2h_state_reset, then decode
 * again).  A model whose path the library chose itself (l2h_model_set_path 0) runs on path 1 from
 * then on, and l2h_model_path / l2h_model_path_reason say so: a GPU that another process shares cannot
 * hold all of path 3's workgroups at once, and every token would end that way.  A model for which
 * path 3 was asked for keeps it.  This sets the bound for path 3 (after finalize).  No counterpart in
 * the reference. */
int l2h_model_set_wait_limit(l2h_model *m, unsigned int spins);
/* l2h_prefill keeps a bf16 copy of the layer matrices (2 bytes per weight, made at its first call
 * when that fits beside 2 GiB of free device memory) and multiplies from it; on = 0 makes it
 * expand the quantized blocks inside the product kernel on every call instead (no extra memory,
 * slower).  With this library's own product kernels (l2h_model_set_prefill_library 0) the results are
 * the same bit for bit.  Default 1.  No counterpart in the reference. */
int l2h_model_set_prefill_copy(l2h_model *m, int on);
/* The products of l2h_prefill that have no arithmetic behind them (q | k | v; wo and w2, whose residual add is the
 * product's beta = 1) go through hipBLASLt, ROCm's GEMM library, when the bf16 copy above exists and the library can be
 * opened at run time (on = 1, the default; the environment variable L2H_PF_LIBRARY=0 has the effect of on = 0); w1 | w3
 * with SwiGLU, the attention and everything else stay with this library's kernels.  on = 0: this library's product
 * kernels throughout.  Same operands (bf16) and fp32 sums either way; the order of the sums differs, so results agree
 * to rounding, not bit for bit.  Takes effect at the next l2h_prefill (the copy's layout is rewritten, a few ms).
 * l2h_model_prefill_library: 1 if the last l2h_prefill ran those products through hipBLASLt.  No counterpart in the
 * reference (matmul! on a matrix of activations is BLAS there too: src/matmul.jl:3-11 for dense matrices). */
int l2h_model_set_prefill_library(l2h_model *m, int on);
int l2h_model_prefill_library(l2h_model *m);
/* RunState(config) (src/inference.jl:88-100): checks every tensor is present, allocates
 * activations and the zeroed KV cache, records the per-token launch sequence. */
int l2h_model_finalize(l2h_model *m);
/* zero the KV cache (a fresh RunState, src/inference.jl:334) */
int l2h_state_reset(l2h_model *m);
/* Write / read n consecutive cache rows of one layer from position pos0: k and v are
 * [n][kv_dim] fp32 (keys already rotated).  The reference fills
 * kv.key_cache[:, :, pos] / kv.value_cache[pos, :, :] (src/inference.jl:259-260). */
int l2h_kv_write(l2h_model *m, int layer, int pos0, int n, const float *k, const float *v);
int l2h_kv_read(l2h_model *m, int layer, int pos0, int n, float *k, float *v);

/* transformer!(token, pos, config, state, weights) (src/inference.jl:222-315).
 * logits (vocab floats) and argmax may each be NULL. argmax is the first maximal index
 * (Julia's argmax, src/inference.jl:360). */
int l2h_forward(l2h_model *m, int token, int pos, float *logits, int32_t *argmax);
/* The loop of sample() at temperature 0 on token ids (src/inference.jl:349-386):
 * feeds prompt[0..n_prompt) from position pos0, then generates n_new tokens greedily;
 * the host is not in the loop.  out gets the n_new ids; last_logits may be NULL. */
int l2h_generate_greedy(l2h_model *m, const int32_t *prompt, int n_prompt, int pos0, int n_new, int32_t *out,
                        float *last_logits);
/* Same, and reports the device time of the n_new generation steps (prompt excluded),
 * measured with HIP events on the context's stream. */
int l2h_generate_greedy_timed(l2h_model *m, const int32_t *prompt, int n_prompt, int pos0, int n_new,
                              int32_t *out, float *decode_ms);
/* Batched prompt pass: positions pos0..pos0+n-1 of tokens[0..n) in one go.  The reference has no
 * batched path; the result is defined as what calling transformer! (src/inference.jl:222-315) for
 * these positions in turn leaves behind: the K/V cache rows pos0..pos0+n-1 of every layer, the
 * logits of the last position (last_logits, may be NULL) and their argmax (next_token, may be
 * NULL).  Matrix products run as bf16 x bf16 -> fp32 on the matrix cores (weights dequantized with
 * the reference's fp32 expressions, then rounded to bf16; float activations, no q8_K step), so the
 * result matches the per-token path to bf16 accuracy, not bit for bit.  Positions before pos0 must
 * already be in the cache.  Decoding continues with l2h_generate_greedy(&next, 1, pos0+n, ...).
 * Needs head size 32/64/96/128, dim and hidden_dim multiples of 8, w1 and w3 of one type. */
int l2h_prefill(l2h_model *m, const int32_t *tokens, int n, int pos0, float *last_logits, int32_t *next_token);
/* The temperature branch of sample() (src/inference.jl:363-367) on the logits the last step left on
 * the device: logits ./= temperature, softmax!, then wsample's walk with the caller's uniform number
 * u in [0, 1) in place of the global RNG: token = first index whose cumulative probability reaches
 * u * sum(p).  probs (vocab floats, may be NULL) receives the probabilities.  temperature > 0. */
int l2h_sample(l2h_model *m, float temperature, float u, int32_t *token, float *probs);
/* Copies an activation of the last forward call: which = 0 x, 1 xb, 2 q (rotated), 5 hb,
 * 6 logits (RunState fields, src/inference.jl:72-86; k and v go straight into the cache). */
int l2h_state_read(l2h_model *m, int which, float *host, int64_t n);

/* ---- single operators (each is the device form of one reference function) ----------- */
/* quantize x[n] (n % 256 == 0) to block_q8_K records (src/kquants.jl:37-42: f32 d,
 * i8 qs[256], i16 bsums[16]; 292 bytes each) with llama.cpp's quantize_row_q8_K rule.
 * The library holds two forms of this quantizer (a block per wavefront in the per-phase
 * kernels, four blocks per wavefront in the streaming kernel); the call runs both and
 * fails with L2H_EHIP if their outputs differ.  x must be finite (L2H_EINVAL otherwise: the
 * rule's "first element of largest magnitude" is undefined for a NaN); inside the decode
 * kernels a non-finite activation gives unspecified quants but no fault. */
int l2h_quantize_q8k(l2h_ctx *ctx, const float *x, int64_t n, void *out_blocks);
/* dequantize!(y, x) (src/kquants.jl:44,70,186,322): nb blocks -> 256*nb floats
 * (F32: nb elements copied). */
int l2h_dequantize(l2h_ctx *ctx, int ggml_type, const void *blocks, int64_t nb, float *y);
/* matmul!(y, A, x) (src/matmul.jl:3-23): uploads A (ne0 x ne1, as set_tensor), runs the
 * same matvec kernel the model uses (k-quant: on q8_K-quantized x; F32: on x), y[ne1].
 * I_sc / I_min (may be NULL; k-quant only) receive, per (row, super-block), the integer
 * sums the kernel formed: [ne1][ne0/256] int32 each.  k-quant: ne0 <= 16384. */
int l2h_matmul(l2h_ctx *ctx, int ggml_type, const void *A, int64_t ne0, int64_t ne1, const float *x, float *y,
               int32_t *I_sc, int32_t *I_min);
/* matmul!(y, A, x) (src/matmul.jl:13-23 as transformer! calls it, src/inference.jl:247-249, 281, 291-292,
 * 302, 312) with A one of the model's resident matrices: role L2H_TOK_EMB, L2H_OUTPUT or L2H_WQ..L2H_W3 of
 * `layer` (ignored for the first two).  x[ne0] and y[ne1] are host arrays.  Nothing is uploaded but x: this is
 * the seam at which the reference's own transformer! runs on device-resident weights (a matrix type whose
 * matmul! method calls this). */
int l2h_model_matmul(l2h_model *m, int role, int layer, const float *x, float *y);
/* rmsnorm!(o, x, weight) (src/inference.jl:102-110). o may alias x. n <= 15360. */
int l2h_rmsnorm(l2h_ctx *ctx, float *o, const float *x, const float *weight, int64_t n);
/* rmsnorm! followed by q8_K quantization of the result, exactly as the matvec kernels do it in
 * their prologue (src/inference.jl:244 then the activation quantizer); n % 256 == 0. */
int l2h_rmsnorm_q8k(l2h_ctx *ctx, const float *x, const float *weight, int64_t n, void *out_blocks);
/* rope!(x, pos, config) (src/inference.jl:112-167) on x[n_heads][head_size]. */
int l2h_rope(l2h_ctx *ctx, float *x, int head_size, int n_heads, int pos, float freq_base, int neox);
/* softmax!(x) (src/inference.jl:169-174) */
int l2h_softmax(l2h_ctx *ctx, float *x, int64_t n);
/* attention_weights! + scale + softmax! + combine_values! (src/inference.jl:176-220,
 * 266-278) for one position: q[n_heads][hs]; kc, vc [(pos+1)][n_kv_heads*hs];
 * out[n_heads][hs]. */
int l2h_attention(l2h_ctx *ctx, float *out, const float *q, const float *kc, const float *vc, int head_size,
                  int n_heads, int n_kv_heads, int pos);
/* hb = hb * sigmoid(hb) .* hb2 (src/inference.jl:295-299) */
int l2h_swiglu(l2h_ctx *ctx, float *hb, const float *hb2, int64_t n);
/* argmax(logits), first maximal index, 0-based (src/inference.jl:360) */
int l2h_argmax(l2h_ctx *ctx, const float *x, int64_t n, int32_t *out);

/* The same argmax for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  x_dev (n floats) and out_dev (one
 * int32) are DEVICE pointers owned by the caller; the call allocates nothing, enqueues its two kernels on
 * the context's stream and returns without waiting (l2h_sync waits).  The kernels' intermediate keys live
 * in a 2 KiB array inside the library's device image, one copy per GPU, held until the process ends:
 * calls that overlap on one GPU (two contexts on one device) race on it.  n above
 * L2H_ARGMAX_NOALLOC_MAX_N is L2H_EINVAL. */
#define L2H_ARGMAX_NOALLOC_MAX_N ((int64_t)1 << 30)
int l2h_argmax_noalloc(l2h_ctx *ctx, const float *x_dev, int64_t n, int32_t *out_dev);

/* ---- measurement -------------------------------------------------------------------- */
/* Launches the model's matvec for `role` on every layer in turn, `iters` times over,
 * between two HIP events on the context's stream; *avg_us = mean time of one launch,
 * *bytes = weight bytes one launch streams (GGUF block bytes x blocks).  role = L2H_W1
 * times the fused w1+w3 launch, L2H_WQ the fused q/k/v launch.
 * The launches are the model's own and write where a decode step writes: the call leaves the
 * RunState (residual stream, position, cache row 0 of every layer) in an undefined state.  Call
 * l2h_state_reset and feed the prompt again before decoding on. */
int l2h_profile_matvec(l2h_model *m, int role, int iters, float *avg_us, int64_t *bytes);
/* plain device-to-device read of n bytes, timed with HIP events: the measured streaming
 * ceiling the roofline fractions can be restated against. */
int l2h_profile_stream_read(l2h_ctx *ctx, int64_t n_bytes, int iters, float *avg_us);

/* ---- synthetic weights (host code; the reference has no quantizer) ------------------- */
/* out[i] = sigma * N(0,1) from a counter-based generator keyed by (seed, stream, offset+i):
 * any slice of any tensor can be regenerated alone. */
int l2h_synth_normal(uint64_t seed, uint64_t stream, int64_t offset, int64_t n, float sigma, float *out,
                     int nthreads);
/* fp32 -> q4_K / q5_K / q6_K super-blocks (n % 256 == 0), llama.cpp block structure:
 * the output bytes are valid GGUF blocks that dequantize! decodes. */
int l2h_quantize_weights(int ggml_type, const float *x, int64_t n, void *out_blocks, int nthreads);

#ifdef __cplusplus
}
#endif
#endif /* L2H_H */

// Internal declarations shared by the kernel files and the C-ABI layer of libl2hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <string>
#include <vector>

#include "l2h.h"

#define QK_K 256

// ------------------------------------------------------------------------------------------
// Device-resident weight tensor.  One allocation per tensor, split into field streams
// (structure-of-arrays over the GGUF super-blocks) so that a wavefront reads every stream
// with 16-byte lane loads over contiguous memory:
//   F32   f32 [ne1][ne0]
//   Q4_K  hdr  16 B/block  = {f16 d, f16 dmin, u8 scales[12]}  (the block's first 16 bytes)
//         qs  128 B/block
//   Q5_K  hdr  16 B/block, qh 32 B/block, qs 128 B/block
//   Q6_K  ql  128 B/block, qh 64 B/block,
//         sc   16 B/block  (int8 scales, byte (4*(2n+hh)+g) <- original byte (8n+hh+2g), so
//                           the four scales one lane needs are one aligned dword)
//         d     2 B/block  (f16)
// Blocks keep GGUF order: block (row, b) has index row*nb + b in every stream.
// ------------------------------------------------------------------------------------------
struct DevTensor {
    int type = -1;
    int64_t ne0 = 0, ne1 = 0, nb = 0;  // nb = ne0/256 super-blocks per row (k-quants)
    void *base = nullptr;
    int64_t bytes = 0;                  // allocation size
    int64_t gguf_bytes = 0;             // bytes the tensor occupies in a GGUF file
    bool slab_member = false;           // lives inside a per-role slab (owned by layer 0's tensor)
    int64_t layer_stride = 0;           // bytes from this tensor to the same tensor of the next layer (slab), or 0
    // stream pointers into base
    const uint4 *hdr = nullptr;         // Q4_K, Q5_K
    const uint8_t *qs = nullptr;        // Q4_K, Q5_K (128 B/block); Q6_K: ql
    const uint8_t *qh = nullptr;        // Q5_K (32 B/block); Q6_K (64 B/block)
    const uint32_t *sc6 = nullptr;      // Q6_K permuted scales, 4 dwords/block
    const uint16_t *d6 = nullptr;       // Q6_K f16 d
    const float *f32 = nullptr;         // F32
};

// q8_K activations on the device: structure-of-arrays over the block_q8_K fields.
struct Q8Dev {
    int8_t *qs;      // [n]
    int16_t *bsums;  // [n/16]
    float *d;        // [n/256]
};

// Per-sequence control block in device memory, read and advanced by the kernels so that
// a recorded launch sequence can be replayed for every token without host involvement.
struct DecodeCtl {
    int32_t token;      // input token of the current step
    int32_t pos;        // 0-based position of the current step
    int32_t step;       // index of the current step within the generate call
    int32_t n_prompt;   // prompt length of the generate call
    int32_t last_argmax;
    int32_t n_out;      // number of generated ids written so far
    int32_t pad[2];
};

// One matvec launch covers up to 3 weight matrices of one type that consume the same input
// vector, with a fused prologue (how the activations reach LDS) and epilogue.
enum { PRO_Q8 = 0, PRO_QUANT = 1, PRO_RMSNORM = 2 };
enum { EPI_STORE = 0, EPI_RESID = 1, EPI_SWIGLU = 2, EPI_ROPE_KV = 3 };
enum { SEG_Q = 0, SEG_K = 1, SEG_V = 2 };
struct PhaseArgs {
    DevTensor w[3];
    float *y[3];           // STORE/RESID: output rows of each segment; SWIGLU: y[0] = hb; ROPE_KV: q rows
    int nseg;
    int seg_roles;         // ROPE_KV: SEG_Q / SEG_K / SEG_V of segment s in bits 2s, 2s+1
    // filled by k_matvec: logical rows in total and per workgroup (even), tile shape
    int64_t n_rows;
    int rows_per_wg, rt, st, ntpr;
    int max_grid;          // workgroups to use at most (number of compute units)
    Q8Dev xq;              // PRO_Q8: quantized input
    const float *xf;       // PRO_QUANT / PRO_RMSNORM: fp32 input
    const float *normw;    // PRO_RMSNORM: norm weights
    int64_t normw_stride;  // bytes to the next layer's norm weights
    int64_t cache_stride;  // bytes to the next layer's kc / vc
    const float *resid;    // EPI_RESID: y = resid + result (may alias y)
    // EPI_ROPE_KV
    const float *rope_cs;  // [hs/2][2] cos, sin of the current position
    double *qd;            // rotated q widened to fp64
    float *kc, *vc;        // this layer's caches
    const DecodeCtl *ctl;
    int hs, seq_len, neox;
    int kv16;              // the caches hold fp16 elements (kc, vc are then byte addresses of such arrays)
    // debug: per (row, block) integer sums (EPI_STORE only), or nullptr
    int32_t *dbg_isc, *dbg_imin;
    int64_t dbg_row0[3];
#ifdef L2H_TIMELINE
    long long *timeline;   // profiling build only: [workgroup][8] wall-clock stamps
#endif
};

// State of the grid-wide barrier of the persistent decode kernel: 16 arrival counters (one per
// 16 workgroups) feeding a root counter, and 8 copies of the release flag; every word sits in
// its own 128-byte line.  Counters only grow: barrier number g completes when they reach g times
// their arrival count.
struct GridBar {
    unsigned long long count[17 * 16];
    unsigned long long flag[8 * 16];
    unsigned int abort;  // set when a workgroup gave up waiting; the kernel then drains
    unsigned int pad[31];
};

// Arguments of the persistent decode kernel (one launch = one token).
struct MegaArgs {
    GridBar *bar;
    unsigned long long gen0;  // barriers completed by earlier launches
    DevTensor emb;
    DecodeCtl *ctl;
    const int32_t *prompt;
    float *x, *xb, *q, *rope_cs, *logits;
    float *kc, *vc;  // layer 0; layer l at + l * cache_layer_elems
    int64_t cache_layer_elems;
    unsigned long long *argmax_partial;  // one slot per workgroup
    int32_t *out_tokens;
    int max_out;
    float theta_scale;
    int hs, n_heads, n_kv_heads, seq_len, n_layers, dim, vocab;
    unsigned int spin_limit;  // polls before a barrier wait gives up
#ifdef L2H_TIMELINE
    long long *timeline;      // profiling build only: [workgroup][64] wall-clock stamps of the first phases
#endif
};

// Streaming decode kernel (k_flow.hip): geometry of one matvec phase, and the kernel's arguments.
struct FlowGeom {
    int n_rows;  // logical rows
    int rpw;     // rows per workgroup (even)
    int ppr;     // pieces per row; 0: rows of K = 1024 (2 i + 1) inputs end in the middle of a piece and go in pairs of
                 // K / 1024 pieces, the pair's middle piece holding the end of the even row and the start of the odd one
    int K;       // input length
};
struct FlowArgs {
    const unsigned char *stream;  // per-wavefront weight streams
    const int64_t *wave_off;      // [grid * 16] byte offset of each wavefront's stream
    // activations as {fp32 value, epoch} words
    unsigned long long *q, *kcur, *vcur, *amax;
    // long-cache attention: per head and member workgroup the run's largest score [heads][G], its sum of
    // exponentials [heads][G][2], its partial value sums [heads][G][hs][2]
    unsigned long long *att_x;
    // activations as bare fp32 words, 0xFFFFFFFF = not written yet: the residual stream in two buffers,
    // attention outputs [2][dim] and SwiGLU outputs [2][hidden] (the pairs alternate from layer to layer)
    unsigned int *x_a, *x_b, *xo, *hbw;
    float *kc, *vc, *logits;
    const float *rms_att, *rms_ffn, *rms_final;
    int64_t norm_stride;  // floats between the norm weights of consecutive layers
    int64_t cache_layer_elems;
    DevTensor emb;
    DecodeCtl *ctl;
    const int32_t *prompt;
    int32_t *out_tokens;
    int max_out;
    unsigned int gen0, spin_limit;
    unsigned int *abort_flag;
    unsigned long long *tokw;  // {token, epoch} in eight copies, 16 words apart: the token of a launch's next step, from workgroup 0 to all
    int dim, hidden, hs, n_heads, n_kv_heads, kv_dim, seq_len, n_layers, vocab, neox;
    int kv16;     // the KV cache holds fp16 elements (typed-piece instantiation of the kernel only)
    int dim_pad;  // dim rounded up to whole pieces (2048): rows of dim inputs are padded with zero super-blocks in the streams
    float theta_scale;
    FlowGeom qkv, wo, w13, w2, cls;
    // layer matrices that are not all q4_K: typed pieces (k_flow.hip), the types of every wavefront's first pieces
    int mixed;
    const unsigned int *wave_types;  // [grid * 16]
    // a model of fp32 matrices (llama2.c files): no streams, the rows are read where the tensors lie.
    // f_w: wq, wk, wv, wo, w1, w3, w2 of layer 0 and the classifier; f_stride: floats from a layer's tensor to the next layer's
    int f32;
    const float *f_w[8];
    int64_t f_stride[8];
#ifdef L2H_TIMELINE
    long long *timeline;  // profiling build only: [workgroup][64] wall-clock stamps of the first phases
#endif
};
// layer_types: per layer the ggml types of wq, wk, wv, wo, w1, w2, w3 (seven numbers a layer)
bool k_flow_plan(FlowArgs &a, const int *layer_types, int n_layer_types, int cls_type, int grid, std::string *why);
int64_t k_flow_offsets(const FlowArgs &a, int cls_type, int grid, std::vector<int64_t> &off);
// Where every typed piece goes (a.mixed): per wavefront the stream's offset, the index of its first piece in the
// per-piece tables, where its classifier pieces start, the types of its first pieces; per piece the byte offset in
// the wavefront's stream and the tag (own type | type of the piece FLOWM_D places on << 8, 3 = none).
struct FlowTypedTables {
    std::vector<int64_t> wave_off, piece_base, cls_off, piece_off;
    std::vector<uint16_t> piece_tag;
    std::vector<unsigned int> wave_types;
    int64_t total = 0;
};
void k_flow_typed_tables(const FlowArgs &a, const int *layer_types, int cls_type, int grid, FlowTypedTables &t);
struct FlowTypedDev {  // the same on the device, for the repack kernel (null for a model of q4_K layers)
    const int64_t *piece_base = nullptr, *cls_off = nullptr, *piece_off = nullptr;
    const uint16_t *piece_tag = nullptr;
};
// kind 0 q|k|v, 1 wo, 2 w1|w3, 3 w2 (of `layer`), 4 classifier; w: the phase's tensors
hipError_t k_flow_repack(hipStream_t s, const FlowArgs &a, unsigned char *stream, const int64_t *wave_off_dev, int kind,
                         int layer, const DevTensor *w, int nw, int grid, int cls_type, const FlowTypedDev &typed);
hipError_t k_flow_bind(hipStream_t s, const FlowArgs &a);
// one launch runs n_tok steps of the token loop; the epochs of the launch start at gen0 and take 5 * n_layers + 2 per step
// form: 0 q4_K pieces, 1 typed pieces, 2 typed pieces and rows that end inside a piece (flow_form)
hipError_t k_flow_launch(hipStream_t s, unsigned int gen0, int n_tok, int cls_type, int grid, int form);
bool k_flow_fits(int cls_type, int grid, int n_cu, int form);
inline int flow_form(const FlowArgs &a) { return a.mixed ? (a.qkv.ppr == 0 ? 2 : 1) : 0; }

// ---- launchers (kernel files) ----------------------------------------------------------------
// Each returns hipGetLastError() of its launch.
hipError_t k_repack(hipStream_t s, const DevTensor &t, const void *raw_dev, bool inverse, void *raw_out);
hipError_t k_embed(hipStream_t s, const DevTensor &emb, const DecodeCtl *ctl, const int32_t *prompt, float *x,
                   float *rope_cs, int head_size, float theta_scale);
hipError_t k_dequant(hipStream_t s, const DevTensor &t, int64_t row0, int64_t nrows, float *y);
hipError_t k_swiglu(hipStream_t s, float *hb, const float *hb2, int n);
hipError_t k_matvec(hipStream_t s, PhaseArgs a, int pro, int epi);
// fills the row split and tile shape of a phase for a grid of at most a.max_grid workgroups; returns the grid
int k_matvec_plan(PhaseArgs &a, int epi);
// persistent decode kernel: supported for the given tensor types?  LDS bytes it needs; launch
bool k_mega_supported(int t_qkv, int t_wo, int t_w13, int t_w2, int t_out);
size_t k_mega_lds_bytes(const MegaArgs &g, const PhaseArgs *ph);
// ph: q/k/v, wo, w1+w3, w2 of layer 0 (later layers are addressed by stride) and the classifier
hipError_t k_mega_bind(hipStream_t s, const PhaseArgs *ph);
hipError_t k_mega_launch(hipStream_t s, const MegaArgs &g, int t_qkv, int t_wo, int t_w13, int t_w2, int t_out, int grid,
                         size_t lds);
hipError_t k_stage_dump(hipStream_t s, const float *x, const float *normw, int64_t n, int pro, Q8Dev q8_out, float *f32_out);
// the same quantization in the streaming decode kernel's form (four blocks per wavefront)
hipError_t k_quantize_rows16(hipStream_t s, const float *x, int64_t n, Q8Dev q8_out);
hipError_t k_rope_only(hipStream_t s, float *x, int head_size, int n_heads, int pos, float theta_scale, int neox);
// kv16: the caches hold fp16 elements (needs head_size <= 128, a multiple of 32)
hipError_t k_attention(hipStream_t s, const double *qd, const float *kc, const float *vc, float *att, double *pd,
                       double *part, float *out, const DecodeCtl *ctl, int head_size, int n_heads,
                       int n_kv_heads, int seq_len, int kv16);
// one launch for scores + softmax + values; needs head_size*8 + seq_len*12 + 8 KiB of LDS <= 64 KiB
hipError_t k_attention_fused(hipStream_t s, const float *q, float *xb, const float *kc, const float *vc,
                             const DecodeCtl *ctl, int head_size, int n_heads, int n_kv_heads, int seq_len);
hipError_t k_softmax(hipStream_t s, float *x, int64_t n);
hipError_t k_argmax(hipStream_t s, const float *x, int64_t n, int64_t *partial, DecodeCtl *ctl, int32_t *out_tokens,
                    int max_out);
// argmax without allocations: k_noalloc_init once per device (that device current), then k_argmax_noalloc
hipError_t k_noalloc_init(int device);
hipError_t k_argmax_noalloc(hipStream_t s, int device, const float *x_dev, int64_t n, int32_t *out_dev);
hipError_t k_sample(hipStream_t s, const float *logits, int n, float temperature, float u, float *p, int32_t *out);
hipError_t k_kv_layout(hipStream_t s, float *kc, float *vc, float *k_lin, float *v_lin, int pos0, int n, int head_size,
                       int n_kv_heads, int seq_len, bool to_cache, int kv16);
hipError_t k_stream_read(hipStream_t s, const uint4 *p, int64_t n16, uint32_t *sink);
hipError_t k_f32_to_f64(hipStream_t s, const float *x, double *y, int64_t n);

// batched prompt pass (k_prefill.hip); activations travel as bf16 bit patterns
enum { PF_STORE = 0, PF_RESID = 1, PF_SWIGLU = 2 };
hipError_t k_pf_embed(hipStream_t s, const DevTensor &emb, const int32_t *tokens, float *X, int M);
hipError_t k_pf_rope_table(hipStream_t s, float *cs, int pos0, int M, int half, float theta_scale);
hipError_t k_pf_rmsnorm(hipStream_t s, const float *X, const float *w, uint16_t *out, int M, int64_t K);
hipError_t k_pf_rope_scatter(hipStream_t s, const float *raw, const float *cs, uint16_t *Qb, float *kc, float *vc, int M,
                             int pos0, int dim, int kv_dim, int hs, int seq_len, int neox);
hipError_t k_pf_gemm(hipStream_t s, const DevTensor *w, int nseg, int interleave, const uint16_t *wbf, int64_t n_rows_bf,
                     const uint16_t *act, int M, int64_t K, int epi, float *out, int64_t ldo, int64_t out_col0,
                     uint16_t *out_bf, int64_t ldb);
// plain: rows of K bf16 values one after the other (what pf_lt_gemm multiplies from) instead of the product kernels' tiles
hipError_t k_pf_expand(hipStream_t s, const DevTensor *w, int nseg, int interleave, int64_t K, uint16_t *dst,
                       int64_t dst_row0, int pad, int plain);
// hipBLASLt for the plain products of the prompt pass (pf_lt.cpp): D[M][0..N) (fp32, row stride ldd) = X[M][K] W[N][K]^T
// (+ D if accumulate), bf16 operands, fp32 sums.  pf_lt_open returns nullptr, and says why, where the library cannot be used.
// pf_lt_gemm with D == nullptr only prepares the shape (hipErrorNotSupported: the library has no algorithm for it).
struct PfLt;
PfLt *pf_lt_open(std::string *why);
void pf_lt_close(PfLt *lt);
hipError_t pf_lt_gemm(PfLt *lt, hipStream_t s, const uint16_t *W, const uint16_t *X, float *D, int M, int64_t N, int64_t K,
                      int64_t ldd, bool accumulate, std::string *err);
bool k_pf_attention_supported(int hs);
int64_t k_pf_kv_tile_bytes(int hs);
hipError_t k_pf_kv_tiles(hipStream_t s, const float *kc, const float *vc, unsigned char *tiles, int n_tiles,
                         int n_tiles_max, int hs, int n_kv, int seq_len);
hipError_t k_pf_attention(hipStream_t s, const uint16_t *Qb, uint16_t *Att, const unsigned char *tiles, int n_tiles_max,
                          int M, int qpos0, int hs, int n_heads, int n_kv, int dim);

static inline int64_t l2h_gguf_block_bytes(int type) {
    switch (type) {
    case L2H_TYPE_F32: return 4;
    case L2H_TYPE_Q4_K: return 144;
    case L2H_TYPE_Q5_K: return 176;
    case L2H_TYPE_Q6_K: return 210;
    }
    return -1;
}

// number of argmax partial slots
#define L2H_ARGMAX_BLOCKS 256
// timesteps handled per attention work item
#define L2H_ATT_TILE 64

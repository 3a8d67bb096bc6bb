// C ABI of libl2hip.so (declared in include/l2h.h): contexts, device-resident models, the
// recorded per-token launch sequence, single-operator entry points and measurement helpers.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <cmath>

#include <algorithm>
#include <mutex>
#include <string>
#include <vector>

#include "l2h_internal.h"

// ------------------------------------------------------------------------------------------
struct l2h_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    std::string err;
    hipDeviceProp_t prop;
};

static std::string g_create_err;

static int set_err(l2h_ctx *ctx, int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (ctx)
        ctx->err = buf;
    else
        g_create_err = buf;
    return code;
}

#define HIPCHK(ctx, call)                                                                          \
    do {                                                                                           \
        hipError_t e_ = (call);                                                                    \
        if (e_ != hipSuccess)                                                                      \
            return set_err((ctx), L2H_EHIP, "%s:%d: %s failed: %s", __FILE__, __LINE__, #call,     \
                           hipGetErrorString(e_));                                                 \
    } while (0)

static bool is_kquant(int type) {
    return type == L2H_TYPE_Q4_K || type == L2H_TYPE_Q5_K || type == L2H_TYPE_Q6_K;
}
static bool type_ok(int type) { return type == L2H_TYPE_F32 || is_kquant(type); }
// longest input vector of a k-quant matvec: the activation staging of the kernels holds
// STAGE_MAX_ROUNDS (4) q8_K blocks per wavefront, 16 wavefronts
#define L2H_MAX_KQ_INPUT 16384

static int64_t align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

// Lays out the field streams of a tensor inside one allocation (see DevTensor).
static int dev_tensor_alloc(l2h_ctx *ctx, int type, int64_t ne0, int64_t ne1, DevTensor *t) {
    *t = DevTensor();
    t->type = type;
    t->ne0 = ne0;
    t->ne1 = ne1;
    if (type == L2H_TYPE_F32) {
        t->nb = 0;
        t->gguf_bytes = ne0 * ne1 * 4;
        t->bytes = align256(t->gguf_bytes);
        HIPCHK(ctx, hipMalloc(&t->base, (size_t)t->bytes));
        t->f32 = (const float *)t->base;
        return L2H_OK;
    }
    t->nb = ne0 / QK_K;
    const int64_t nblk = t->nb * ne1;
    t->gguf_bytes = nblk * l2h_gguf_block_bytes(type);
    int64_t off_hdr = 0, off_qs = 0, off_qh = 0, off_sc = 0, off_d = 0, total = 0;
    if (type == L2H_TYPE_Q4_K) {
        off_hdr = 0;
        off_qs = align256(nblk * 16);
        total = off_qs + align256(nblk * 128);
    } else if (type == L2H_TYPE_Q5_K) {
        off_hdr = 0;
        off_qh = align256(nblk * 16);
        off_qs = off_qh + align256(nblk * 32);
        total = off_qs + align256(nblk * 128);
    } else {
        off_qs = 0;
        off_qh = align256(nblk * 128);
        off_sc = off_qh + align256(nblk * 64);
        off_d = off_sc + align256(nblk * 16);
        total = off_d + align256(nblk * 2);
    }
    t->bytes = total;
    HIPCHK(ctx, hipMalloc(&t->base, (size_t)total));
    char *b = (char *)t->base;
    if (type != L2H_TYPE_Q6_K) t->hdr = (const uint4 *)(b + off_hdr);
    t->qs = (const uint8_t *)(b + off_qs);
    if (type != L2H_TYPE_Q4_K) t->qh = (const uint8_t *)(b + off_qh);
    if (type == L2H_TYPE_Q6_K) {
        t->sc6 = (const uint32_t *)(b + off_sc);
        t->d6 = (const uint16_t *)(b + off_d);
    }
    return L2H_OK;
}

static void dev_tensor_free(DevTensor *t) {
    if (t->base) (void)hipFree(t->base);
    *t = DevTensor();
}

// host GGUF blocks -> device field streams
static int dev_tensor_upload(l2h_ctx *ctx, DevTensor *t, const void *host) {
    if (t->type == L2H_TYPE_F32) {
        HIPCHK(ctx, hipMemcpy(t->base, host, (size_t)t->gguf_bytes, hipMemcpyHostToDevice));
        return L2H_OK;
    }
    void *raw = nullptr;
    HIPCHK(ctx, hipMalloc(&raw, (size_t)t->gguf_bytes));
    hipError_t e = hipMemcpy(raw, host, (size_t)t->gguf_bytes, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = k_repack(ctx->stream, *t, raw, false, nullptr);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    (void)hipFree(raw);
    if (e != hipSuccess) return set_err(ctx, L2H_EHIP, "tensor upload failed: %s", hipGetErrorString(e));
    return L2H_OK;
}

static int dev_tensor_download(l2h_ctx *ctx, const DevTensor *t, void *host) {
    if (t->type == L2H_TYPE_F32) {
        HIPCHK(ctx, hipMemcpy(host, t->f32, (size_t)t->gguf_bytes, hipMemcpyDeviceToHost));
        return L2H_OK;
    }
    void *raw = nullptr;
    HIPCHK(ctx, hipMalloc(&raw, (size_t)t->gguf_bytes));
    hipError_t e = k_repack(ctx->stream, *t, nullptr, true, raw);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) e = hipMemcpy(host, raw, (size_t)t->gguf_bytes, hipMemcpyDeviceToHost);
    (void)hipFree(raw);
    if (e != hipSuccess) return set_err(ctx, L2H_EHIP, "tensor download failed: %s", hipGetErrorString(e));
    return L2H_OK;
}

// ------------------------------------------------------------------------------------------
// context
// ------------------------------------------------------------------------------------------
extern "C" int l2h_ctx_create(int device, l2h_ctx **out) {
    if (!out) return set_err(nullptr, L2H_EINVAL, "l2h_ctx_create: out is NULL");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0)
        return set_err(nullptr, L2H_ENODEV, "no HIP device: %s", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= n) return set_err(nullptr, L2H_EINVAL, "device %d out of range (0..%d)", device, n - 1);
    l2h_ctx *ctx = new l2h_ctx();
    ctx->device = device;
    e = hipSetDevice(device);
    if (e == hipSuccess) e = hipGetDeviceProperties(&ctx->prop, device);
    if (e == hipSuccess) e = hipStreamCreate(&ctx->stream);
    if (e == hipSuccess) e = k_noalloc_init(device);  // address of this device's copy of the no-allocation scratch array
    if (e != hipSuccess) {
        set_err(nullptr, L2H_EHIP, "context setup failed: %s", hipGetErrorString(e));
        delete ctx;
        return L2H_EHIP;
    }
    if (strncmp(ctx->prop.gcnArchName, "gfx950", 6) != 0) {
        set_err(nullptr, L2H_ENODEV, "device %d is %s; this library is built for gfx950 only", device,
                ctx->prop.gcnArchName);
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return L2H_ENODEV;
    }
    *out = ctx;
    return L2H_OK;
}

extern "C" void l2h_ctx_destroy(l2h_ctx *ctx) {
    if (!ctx) return;
    if (ctx->stream) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipStreamDestroy(ctx->stream);
    }
    delete ctx;
}

extern "C" const char *l2h_last_error(l2h_ctx *ctx) { return ctx ? ctx->err.c_str() : g_create_err.c_str(); }

extern "C" int l2h_sync(l2h_ctx *ctx) {
    if (!ctx) return L2H_EINVAL;
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return L2H_OK;
}

extern "C" int l2h_device_info(l2h_ctx *ctx, char *name, int name_cap, int32_t *n_cu, int64_t *hbm_bytes) {
    if (!ctx) return L2H_EINVAL;
    if (name && name_cap > 0) snprintf(name, (size_t)name_cap, "%s (%s)", ctx->prop.name, ctx->prop.gcnArchName);
    if (n_cu) *n_cu = ctx->prop.multiProcessorCount;
    if (hbm_bytes) *hbm_bytes = (int64_t)ctx->prop.totalGlobalMem;
    return L2H_OK;
}

// ------------------------------------------------------------------------------------------
// model
// ------------------------------------------------------------------------------------------
struct l2h_model;
static l2h_model *g_bound_model = nullptr;  // whose phase arguments the persistent kernel's constant memory holds
static l2h_model *g_flow_bound = nullptr;   // whose arguments the streaming kernel's constant memory holds

struct l2h_model {
    l2h_ctx *ctx = nullptr;
    l2h_config c{};
    int hs = 0, kv_dim = 0;
    float theta_scale = 0.0f;
    DevTensor glob[3];
    std::vector<DevTensor> layer;  // [n_layers][L2H_N_ROLES]
    bool finalized = false;
    // RunState (reference src/inference.jl:72-100) in device memory
    float *x = nullptr, *xb = nullptr, *xb2 = nullptr, *hb = nullptr, *hb2 = nullptr, *q = nullptr, *k = nullptr,
          *v = nullptr, *att = nullptr, *logits = nullptr;
    double *qd = nullptr, *pd = nullptr, *part = nullptr;
    float *rope_cs = nullptr;  // cos/sin of the current position's RoPE angles, [hs/2][2]
    float *kc = nullptr, *vc = nullptr;  // [n_layers] x per-layer cache
    int64_t cache_layer_elems = 0;
    DecodeCtl *ctl = nullptr;
    int32_t *prompt_dev = nullptr, *out_tokens = nullptr;
    int64_t *argmax_partial = nullptr;
    int max_out = 0;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    // persistent decode kernel
    int kv16 = 0;          // 1: the KV cache holds fp16 elements (l2h_model_set_kv_type)
    bool kv_uncached = false;       // the KV cache lives in uncached memory (see l2h_model_finalize)
    int flow_steps_per_launch = 1;  // steps of the token loop per launch of the streaming kernel
    int path_request = 0;  // 0 auto, 1 one kernel per phase, 2 persistent kernel, 3 streaming kernel (2, 3: required)
    bool mega = false;
    PhaseArgs mega_ph[5];  // q/k/v, wo, w1+w3, w2 of layer 0 and the classifier, planned for the persistent grid
    GridBar *bar = nullptr;
    unsigned long long bar_gen = 0;
    int mega_grid = 0;
    size_t mega_lds = 0;
    int mega_types[5] = {0, 0, 0, 0, 0};
#ifdef L2H_TIMELINE
    long long *timeline = nullptr, *timeline2 = nullptr;
#endif
    float *sample_p = nullptr;  // probabilities of the last l2h_sample call
    int32_t *sample_out = nullptr;
    // streaming decode kernel
    bool flow = false;
    FlowArgs flow_args{};
    int flow_grid = 0, flow_cls_type = 0;
    std::string flow_why;  // why the streaming kernel was not chosen (empty if it was, or if it was not asked for)
    unsigned int flow_gen = 1;  // epoch of the next launch's input; 0 is what cleared memory holds
    // batched prompt pass: buffers for pf_cap positions, allocated at the first l2h_prefill
    int pf_cap = 0;
    float *pf_x = nullptr, *pf_raw = nullptr, *pf_cs = nullptr;
    uint16_t *pf_xn = nullptr, *pf_q = nullptr, *pf_att = nullptr, *pf_hb = nullptr;
    int32_t *pf_tok = nullptr;
    unsigned char *pf_kvt = nullptr;  // one layer's K / V^T as bf16 tiles of 32 keys (k_pf_kv_tiles)
    int pf_kvt_tiles = 0;             // tiles per KV head
    // bf16 copy of the layer matrices for the prompt pass: per layer q|k|v rows, wo, w1/w3 rows in turn, w2
    int pf_copy_mode = 1;          // 0 never, 1 when it fits
    bool pf_copy_tried = false;
    uint16_t *pf_wbf = nullptr;
    // the plain products of the prompt pass (q | k | v, wo, w2) through hipBLASLt: asked for (default) / opened / the
    // layout the copy's three matrices have now (plain rows for the library, tiles for the own kernels)
    int pf_library_mode = 1;
    PfLt *pf_lt = nullptr;
    bool pf_lt_tried = false, pf_plain = false;
    std::string pf_lt_why, pf_lt_err;
    int64_t pf_wbf_layer = 0, pf_off_wo = 0, pf_off_w13 = 0, pf_off_w2 = 0;  // elements
    std::vector<void *> allocs;
    std::vector<void *> uc_allocs;  // blocks of the uncached pool (uncached_alloc), handed back with the model

    DevTensor &L(int layer_idx, int role) { return layer[(size_t)layer_idx * L2H_N_ROLES + role]; }
};

static int q8_alloc(l2h_ctx *ctx, int64_t n, Q8Dev *q, std::vector<void *> *track) {
    void *p = nullptr;
    const int64_t o_bs = align256(n), o_d = o_bs + align256(n / 8 + 16);
    HIPCHK(ctx, hipMalloc(&p, (size_t)(o_d + align256(n / 64 + 16))));
    q->qs = (int8_t *)p;
    q->bsums = (int16_t *)((char *)p + o_bs);
    q->d = (float *)((char *)p + o_d);
    if (track) track->push_back(p);
    return L2H_OK;
}

extern "C" int l2h_model_create(l2h_ctx *ctx, const l2h_config *cfg, l2h_model **out) {
    if (!ctx || !cfg || !out) return set_err(ctx, L2H_EINVAL, "l2h_model_create: NULL argument");
    *out = nullptr;
    const l2h_config &c = *cfg;
    if (c.dim <= 0 || c.hidden_dim <= 0 || c.n_layers <= 0 || c.n_heads <= 0 || c.n_kv_heads <= 0 ||
        c.vocab_size <= 0 || c.seq_len <= 0)
        return set_err(ctx, L2H_EINVAL, "config fields must be positive");
    if (c.dim % c.n_heads != 0) return set_err(ctx, L2H_EINVAL, "dim %d not divisible by n_heads %d", c.dim, c.n_heads);
    if (c.n_heads % c.n_kv_heads != 0)
        return set_err(ctx, L2H_EINVAL, "n_heads %d not divisible by n_kv_heads %d", c.n_heads, c.n_kv_heads);
    const int hs = c.dim / c.n_heads;
    if (hs % 4 != 0 || hs > 1024) return set_err(ctx, L2H_EINVAL, "head_size %d must be a multiple of 4, <= 1024", hs);
    l2h_model *m = new l2h_model();
    m->ctx = ctx;
    m->c = c;
    m->hs = hs;
    m->kv_dim = hs * c.n_kv_heads;
    // theta_scale = freq_base ^ (-1/(head_size/2)) in fp32 (reference src/inference.jl:119)
    m->theta_scale = powf(c.rope_freq_base, -(1.0f / (float)(hs / 2)));
    m->layer.resize((size_t)c.n_layers * L2H_N_ROLES);
    *out = m;
    return L2H_OK;
}

static void uncached_release(void *p);

static void model_free_state(l2h_model *m) {
    if (m->exec) (void)hipGraphExecDestroy(m->exec);
    if (m->graph) (void)hipGraphDestroy(m->graph);
    m->exec = nullptr;
    m->graph = nullptr;
    for (void *p : m->allocs) (void)hipFree(p);
    m->allocs.clear();
    for (void *p : m->uc_allocs) uncached_release(p);
    m->uc_allocs.clear();
    m->pf_cap = 0;
    m->pf_wbf = nullptr;
    m->pf_copy_tried = false;
    pf_lt_close(m->pf_lt);
    m->pf_lt = nullptr;
    m->pf_lt_tried = false;
    m->pf_plain = false;
    m->sample_p = nullptr;
    m->sample_out = nullptr;
    m->finalized = false;
}

extern "C" void l2h_model_destroy(l2h_model *m) {
    if (!m) return;
    if (g_bound_model == m) g_bound_model = nullptr;
    if (g_flow_bound == m) g_flow_bound = nullptr;
    (void)hipStreamSynchronize(m->ctx->stream);
    model_free_state(m);
    for (auto &t : m->glob) dev_tensor_free(&t);
    for (auto &t : m->layer) dev_tensor_free(&t);
    delete m;
}

static const char *role_name(int role) {
    static const char *n[] = {"token_embedding_table", "rms_final_weight", "output_weight", "rms_att_weight",
                              "rms_ffn_weight", "wq", "wk", "wv", "wo", "w1", "w2", "w3"};
    return (role >= 0 && role < L2H_N_ROLES) ? n[role] : "?";
}

extern "C" int l2h_model_set_tensor(l2h_model *m, int role, int layer, int type, const void *host, int64_t ne0,
                                    int64_t ne1) {
    if (!m || !host) return set_err(m ? m->ctx : nullptr, L2H_EINVAL, "l2h_model_set_tensor: NULL argument");
    l2h_ctx *ctx = m->ctx;
    if (m->finalized) return set_err(ctx, L2H_ESTATE, "model already finalized");
    if (role < 0 || role >= L2H_N_ROLES) return set_err(ctx, L2H_EINVAL, "role %d out of range", role);
    if (!type_ok(type)) return set_err(ctx, L2H_ETYPE, "tensor type %d not implemented", type);
    if (role >= 3 && (layer < 0 || layer >= m->c.n_layers))
        return set_err(ctx, L2H_EINVAL, "layer %d out of range", layer);
    const l2h_config &c = m->c;
    int64_t e0 = 0, e1 = 0;
    switch (role) {
    case L2H_TOK_EMB:
    case L2H_OUTPUT: e0 = c.dim; e1 = c.vocab_size; break;
    case L2H_RMS_FINAL:
    case L2H_RMS_ATT:
    case L2H_RMS_FFN: e0 = c.dim; e1 = 1; break;
    case L2H_WQ:
    case L2H_WO: e0 = c.dim; e1 = c.dim; break;
    case L2H_WK:
    case L2H_WV: e0 = c.dim; e1 = m->kv_dim; break;
    case L2H_W1:
    case L2H_W3: e0 = c.dim; e1 = c.hidden_dim; break;
    case L2H_W2: e0 = c.hidden_dim; e1 = c.dim; break;
    }
    if (ne0 != e0 || ne1 != e1)
        return set_err(ctx, L2H_EINVAL, "%s: shape (%lld, %lld) does not match config (%lld, %lld)", role_name(role),
                       (long long)ne0, (long long)ne1, (long long)e0, (long long)e1);
    if ((role == L2H_RMS_FINAL || role == L2H_RMS_ATT || role == L2H_RMS_FFN) && type != L2H_TYPE_F32)
        return set_err(ctx, L2H_ETYPE, "%s must be F32", role_name(role));
    if (is_kquant(type) && ne0 % QK_K != 0)
        return set_err(ctx, L2H_EINVAL, "%s: ne0 = %lld is not a multiple of 256", role_name(role), (long long)ne0);
    if (is_kquant(type) && ne0 > L2H_MAX_KQ_INPUT)
        return set_err(ctx, L2H_EINVAL, "%s: a k-quant matrix takes at most %d input features, got %lld", role_name(role),
                       L2H_MAX_KQ_INPUT, (long long)ne0);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevTensor &slot = role < 3 ? m->glob[role] : m->L(layer, role);
    dev_tensor_free(&slot);
    int rc = dev_tensor_alloc(ctx, type, ne0, ne1, &slot);
    if (rc) return rc;
    rc = dev_tensor_upload(ctx, &slot, host);
    if (rc) dev_tensor_free(&slot);
    return rc;
}

extern "C" int l2h_model_set_wait_limit(l2h_model *m, unsigned int spins) {
    if (!m) return L2H_EINVAL;
    if (!m->flow) return set_err(m->ctx, L2H_ESTATE, "the wait limit applies to launch path 3 after finalize");
    m->flow_args.spin_limit = spins;
    if (g_flow_bound == m) g_flow_bound = nullptr;  // the kernel's copy of the arguments is refreshed at the next launch
    return L2H_OK;
}

extern "C" int l2h_model_set_prefill_copy(l2h_model *m, int on) {
    if (!m) return L2H_EINVAL;
    if (on != 0 && on != 1) return set_err(m->ctx, L2H_EINVAL, "on must be 0 or 1");
    m->pf_copy_mode = on;
    return L2H_OK;
}

extern "C" int l2h_model_set_prefill_library(l2h_model *m, int on) {
    if (!m) return L2H_EINVAL;
    if (on != 0 && on != 1) return set_err(m->ctx, L2H_EINVAL, "on must be 0 or 1");
    m->pf_library_mode = on;
    return L2H_OK;
}

extern "C" int l2h_model_prefill_library(l2h_model *m) { return (m && m->pf_wbf && m->pf_copy_mode && m->pf_plain) ? 1 : 0; }

extern "C" int l2h_model_set_kv_type(l2h_model *m, int kv_type) {
    if (!m) return L2H_EINVAL;
    if (m->finalized) return set_err(m->ctx, L2H_ESTATE, "model already finalized");
    if (kv_type != L2H_KV_F32 && kv_type != L2H_KV_F16) return set_err(m->ctx, L2H_EINVAL, "kv_type must be L2H_KV_F32 or L2H_KV_F16");
    m->kv16 = kv_type == L2H_KV_F16;
    return L2H_OK;
}

extern "C" int l2h_model_set_path(l2h_model *m, int path) {
    if (!m) return L2H_EINVAL;
    if (m->finalized) return set_err(m->ctx, L2H_ESTATE, "model already finalized");
    if (path < 0 || path > 3) return set_err(m->ctx, L2H_EINVAL, "path must be 0, 1, 2 or 3");
    m->path_request = path;
    return L2H_OK;
}

extern "C" const char *l2h_model_path_reason(l2h_model *m) {
    if (!m || !m->finalized) return "";
    return m->flow_why.c_str();
}

extern "C" int l2h_model_steps_per_launch(l2h_model *m) { return (m && m->finalized && m->flow) ? m->flow_steps_per_launch : 1; }
extern "C" int l2h_model_path(l2h_model *m) { return (m && m->finalized) ? (m->flow ? 3 : (m->mega ? 2 : 1)) : 0; }

extern "C" int l2h_model_get_tensor(l2h_model *m, int role, int layer, void *host, int64_t host_bytes) {
    if (!m || !host) return set_err(m ? m->ctx : nullptr, L2H_EINVAL, "l2h_model_get_tensor: NULL argument");
    if (role < 0 || role >= L2H_N_ROLES || (role >= 3 && (layer < 0 || layer >= m->c.n_layers)))
        return set_err(m->ctx, L2H_EINVAL, "role/layer out of range");
    DevTensor &t = role < 3 ? m->glob[role] : m->L(layer, role);
    if (t.type < 0) return set_err(m->ctx, L2H_ESTATE, "%s not set", role_name(role));
    if (host_bytes != t.gguf_bytes)
        return set_err(m->ctx, L2H_EINVAL, "buffer is %lld bytes, tensor is %lld", (long long)host_bytes,
                       (long long)t.gguf_bytes);
    return dev_tensor_download(m->ctx, &t, host);
}

// Device memory that bypasses the caches (hipDeviceMallocUncached), for the words that the workgroups of the
// streaming kernel hand to one another: a word stored there is seen by a poll from another XCD sooner than
// through the L2s (measured: 745 instead of 731 tok/s).  Such memory is never given back to the driver, where
// freed blocks have later turned up with stale contents in new allocations: a block goes back to a free list
// and serves the next model of that device.
namespace {
struct UncachedBlock {
    void *p;
    size_t bytes;
    int device;
    bool used;
};
std::mutex g_uc_mu;
std::vector<UncachedBlock> g_uc_blocks;
}  // namespace

static hipError_t uncached_alloc(int device, size_t bytes, void **out) {
    bytes = (bytes + 4095) / 4096 * 4096;
    std::lock_guard<std::mutex> lock(g_uc_mu);
    UncachedBlock *best = nullptr;
    for (UncachedBlock &b : g_uc_blocks)
        if (!b.used && b.device == device && b.bytes >= bytes && (!best || b.bytes < best->bytes)) best = &b;
    if (best) {
        best->used = true;
        *out = best->p;
        return hipSuccess;
    }
    void *p = nullptr;
    const hipError_t e = hipExtMallocWithFlags(&p, bytes, hipDeviceMallocUncached);
    if (e != hipSuccess) return e;
    g_uc_blocks.push_back(UncachedBlock{p, bytes, device, true});
    *out = p;
    return hipSuccess;
}

static void uncached_release(void *p) {
    std::lock_guard<std::mutex> lock(g_uc_mu);
    for (UncachedBlock &b : g_uc_blocks)
        if (b.p == p) b.used = false;
}

template <class T>
static int dalloc(l2h_model *m, T **p, int64_t n, bool zero) {
    void *v = nullptr;
    const size_t bytes = (size_t)std::max<int64_t>(n, 1) * sizeof(T);
    HIPCHK(m->ctx, hipMalloc(&v, bytes));
    m->allocs.push_back(v);
    if (zero) HIPCHK(m->ctx, hipMemset(v, 0, bytes));
    *p = (T *)v;
    return L2H_OK;
}

// the caches of layer l (fp32 or fp16 elements: addressed in bytes)
static float *layer_kc(l2h_model *m, int l) { return (float *)((char *)m->kc + (int64_t)l * m->cache_layer_elems * (m->kv16 ? 2 : 4)); }
static float *layer_vc(l2h_model *m, int l) { return (float *)((char *)m->vc + (int64_t)l * m->cache_layer_elems * (m->kv16 ? 2 : 4)); }

// ---- the per-token launch sequence: transformer! (reference src/inference.jl:222-315) ----------
static PhaseArgs base_args(l2h_model *m) {
    PhaseArgs a{};
    a.max_grid = m->ctx->prop.multiProcessorCount;
    a.ctl = m->ctl;
    a.hs = m->hs;
    a.seq_len = m->c.seq_len;
    a.neox = m->c.rope_is_neox;
    a.rope_cs = m->rope_cs;
    a.qd = m->qd;
    a.normw_stride = m->L(0, L2H_RMS_ATT).layer_stride;
    a.cache_stride = m->cache_layer_elems * (m->kv16 ? 2 : 4);
    a.kv16 = m->kv16;
    return a;
}

// rmsnorm (:244) + q, k, v (:247-249) + rope (:255-256) + cache append (:259-260); tensors
// first..last-1 of {wq, wk, wv} in one launch (they must share a type)
static PhaseArgs make_qkv(l2h_model *m, int l, int first, int last) {
    const DevTensor *w[3] = {&m->L(l, L2H_WQ), &m->L(l, L2H_WK), &m->L(l, L2H_WV)};
    float *y[3] = {m->q, nullptr, nullptr};
    PhaseArgs a = base_args(m);
    a.xf = m->x;
    a.normw = m->L(l, L2H_RMS_ATT).f32;
    a.kc = layer_kc(m, l);
    a.vc = layer_vc(m, l);
    a.nseg = last - first;
    a.seg_roles = 0;
    for (int k = first; k < last; k++) {
        a.w[k - first] = *w[k];
        a.y[k - first] = y[k];
        a.seg_roles |= k << (2 * (k - first));
    }
    return a;
}

static hipError_t launch_qkv(l2h_model *m, int l) {
    const int t[3] = {m->L(l, L2H_WQ).type, m->L(l, L2H_WK).type, m->L(l, L2H_WV).type};
    int i = 0;
    while (i < 3) {  // consecutive tensors of one type share a launch
        int j = i + 1;
        while (j < 3 && t[j] == t[i]) j++;
        hipError_t e = k_matvec(m->ctx->stream, make_qkv(m, l, i, j), PRO_RMSNORM, EPI_ROPE_KV);
        if (e != hipSuccess) return e;
        i = j;
    }
    return hipSuccess;
}

// x += wo * xb (:281-284); the prologue quantizes the attention output
static PhaseArgs make_wo(l2h_model *m, int l) {
    PhaseArgs a = base_args(m);
    a.nseg = 1;
    a.w[0] = m->L(l, L2H_WO);
    a.y[0] = m->x;
    a.resid = m->x;
    a.xf = m->xb;
    return a;
}
static hipError_t launch_wo(l2h_model *m, int l) {
    return k_matvec(m->ctx->stream, make_wo(m, l), PRO_QUANT, EPI_RESID);
}

// rmsnorm (:287) + w1, w3 (:291-292) + SwiGLU (:295-299) -> hb
static PhaseArgs make_w13(l2h_model *m, int l) {
    PhaseArgs a = base_args(m);
    a.xf = m->x;
    a.normw = m->L(l, L2H_RMS_FFN).f32;
    a.nseg = 2;
    a.w[0] = m->L(l, L2H_W1);
    a.w[1] = m->L(l, L2H_W3);
    a.y[0] = m->hb;
    return a;
}
static hipError_t launch_w13(l2h_model *m, int l) {
    hipStream_t s = m->ctx->stream;
    PhaseArgs a = make_w13(m, l);
    if (a.w[0].type == a.w[1].type) return k_matvec(s, a, PRO_RMSNORM, EPI_SWIGLU);
    // different types: two launches, then the stand-alone SwiGLU
    const DevTensor w3 = a.w[1];
    a.nseg = 1;
    hipError_t e = k_matvec(s, a, PRO_RMSNORM, EPI_STORE);
    if (e != hipSuccess) return e;
    a.w[0] = w3;
    a.y[0] = m->hb2;
    e = k_matvec(s, a, PRO_RMSNORM, EPI_STORE);
    if (e != hipSuccess) return e;
    return k_swiglu(s, m->hb, m->hb2, m->c.hidden_dim);
}

// x += w2 * hb (:302-305)
static PhaseArgs make_w2(l2h_model *m, int l) {
    PhaseArgs a = base_args(m);
    a.nseg = 1;
    a.w[0] = m->L(l, L2H_W2);
    a.y[0] = m->x;
    a.resid = m->x;
    a.xf = m->hb;
    return a;
}
static hipError_t launch_w2(l2h_model *m, int l) {
    return k_matvec(m->ctx->stream, make_w2(m, l), PRO_QUANT, EPI_RESID);
}

// final rmsnorm (:309) + classifier (:312)
static PhaseArgs make_output(l2h_model *m) {
    PhaseArgs a = base_args(m);
    a.nseg = 1;
    a.w[0] = m->glob[L2H_OUTPUT];
    a.y[0] = m->logits;
    a.xf = m->x;
    a.normw = m->glob[L2H_RMS_FINAL].f32;
    return a;
}
static hipError_t launch_output(l2h_model *m) {
    return k_matvec(m->ctx->stream, make_output(m), PRO_RMSNORM, EPI_STORE);
}

// Moves the per-layer tensors of each role into one slab per role, layer l at base + l * stride,
// so that a kernel can address any layer from the layer-0 pointers.
static int rehome_layers(l2h_model *m) {
    l2h_ctx *ctx = m->ctx;
    const int L = m->c.n_layers;
    for (int role = 3; role < L2H_N_ROLES; role++) {
        const DevTensor &t0 = m->L(0, role);
        bool same = true;
        for (int l = 1; l < L; l++) same = same && m->L(l, role).type == t0.type && m->L(l, role).bytes == t0.bytes;
        if (!same) continue;  // mixed types across layers: tensors stay where they are
        char *slab = nullptr;
        HIPCHK(ctx, hipMalloc((void **)&slab, (size_t)t0.bytes * L));
        for (int l = 0; l < L; l++) {
            DevTensor &t = m->L(l, role);
            char *nb = slab + (int64_t)l * t.bytes;
            HIPCHK(ctx, hipMemcpy(nb, t.base, (size_t)t.bytes, hipMemcpyDeviceToDevice));
            const char *ob = (const char *)t.base;
#define MOVE(F) if (t.F) t.F = (decltype(t.F))(nb + ((const char *)t.F - ob))
            MOVE(hdr); MOVE(qs); MOVE(qh); MOVE(sc6); MOVE(d6); MOVE(f32);
#undef MOVE
            (void)hipFree(t.base);
            t.base = l == 0 ? (void *)slab : nullptr;  // the slab is freed through layer 0
            t.slab_member = true;
            t.layer_stride = t.bytes;
        }
    }
    return L2H_OK;
}

// ---- persistent decode kernel: plan + launch -------------------------------------------------
static MegaArgs mega_args(l2h_model *m) {
    MegaArgs g{};
    g.bar = m->bar;
    g.gen0 = m->bar_gen;
    g.emb = m->glob[L2H_TOK_EMB];
    g.ctl = m->ctl;
    g.prompt = m->prompt_dev;
    g.x = m->x;
    g.xb = m->xb;
    g.q = m->q;
    g.rope_cs = m->rope_cs;
    g.logits = m->logits;
    g.kc = m->kc;
    g.vc = m->vc;
    g.cache_layer_elems = m->cache_layer_elems;
    g.argmax_partial = (unsigned long long *)m->argmax_partial;
    g.out_tokens = m->out_tokens;
    g.max_out = m->max_out;
    g.theta_scale = m->theta_scale;
    g.hs = m->hs;
    g.n_heads = m->c.n_heads;
    g.n_kv_heads = m->c.n_kv_heads;
    g.seq_len = m->c.seq_len;
    g.n_layers = m->c.n_layers;
    g.dim = m->c.dim;
    g.vocab = m->c.vocab_size;
    g.spin_limit = 1u << 22;
#ifdef L2H_TIMELINE
    g.timeline = m->timeline;
#endif
    return g;
}

// Decides whether this model can run on the persistent kernel and, if so, builds its plan.
static int mega_setup(l2h_model *m) {
    l2h_ctx *ctx = m->ctx;
    const l2h_config &c = m->c;
    m->mega = false;
    // automatic choice: the per-phase recording, which is the faster of the two at present
    if (m->path_request != 2) return L2H_OK;
    const char *why = nullptr;
    const int t_qkv = m->L(0, L2H_WQ).type, t_wo = m->L(0, L2H_WO).type, t_w13 = m->L(0, L2H_W1).type,
              t_w2 = m->L(0, L2H_W2).type, t_out = m->glob[L2H_OUTPUT].type;
    for (int l = 0; l < c.n_layers && !why; l++) {
        if (m->L(l, L2H_WQ).type != t_qkv || m->L(l, L2H_WK).type != t_qkv || m->L(l, L2H_WV).type != t_qkv ||
            m->L(l, L2H_WO).type != t_wo || m->L(l, L2H_W1).type != t_w13 || m->L(l, L2H_W3).type != t_w13 ||
            m->L(l, L2H_W2).type != t_w2)
            why = "tensor types differ between layers or inside a fused launch";
    }
    if (!why && !k_mega_supported(t_qkv, t_wo, t_w13, t_w2, t_out)) why = "no kernel for this combination of tensor types";
    if (!why && std::max(c.dim, c.hidden_dim) > 16384) why = "activation vector longer than 16384";
    const int grid = ctx->prop.multiProcessorCount;
    if (!why) {
        PhaseArgs a[5] = {make_qkv(m, 0, 0, 3), make_wo(m, 0), make_w13(m, 0), make_w2(m, 0), make_output(m)};
        const int epi[5] = {EPI_ROPE_KV, EPI_RESID, EPI_SWIGLU, EPI_RESID, EPI_STORE};
        for (int k = 0; k < 5; k++) {
            a[k].max_grid = grid;
            if (k_matvec_plan(a[k], epi[k]) <= 0) why = "phase cannot be planned";
            m->mega_ph[k] = a[k];
        }
        if (m->L(0, L2H_RMS_ATT).layer_stride != m->L(0, L2H_RMS_FFN).layer_stride) why = "norm weight slabs differ";
    }
    size_t lds = 0;
    if (!why) {
        MegaArgs g = mega_args(m);
        lds = k_mega_lds_bytes(g, m->mega_ph);
        if (lds > 64 * 1024) why = "needs more than 64 KiB of LDS (sequence too long for the one-head-per-workgroup attention)";
    }
    if (why) {
        if (m->path_request == 2) return set_err(ctx, L2H_EINVAL, "persistent kernel not available: %s", why);
        return L2H_OK;
    }
    int rc;
    if ((rc = dalloc(m, &m->bar, 1, true))) return rc;
    m->bar_gen = 0;
    m->mega_grid = grid;
    m->mega_lds = lds;
    m->mega_types[0] = t_qkv;
    m->mega_types[1] = t_wo;
    m->mega_types[2] = t_w13;
    m->mega_types[3] = t_w2;
    m->mega_types[4] = t_out;
#ifdef L2H_TIMELINE
    if ((rc = dalloc(m, &m->timeline, (int64_t)grid * 64, true))) return rc;
    if ((rc = dalloc(m, &m->timeline2, (int64_t)grid * 8, true))) return rc;
    {
        const char *ph = getenv("L2H_TL_PHASE");
        m->mega_ph[ph ? atoi(ph) : 2].timeline = m->timeline2;
    }
#endif
    m->mega = true;
    return L2H_OK;
}

// Builds the per-wavefront weight streams and the tagged activation buffers of the streaming kernel.
static int flow_setup(l2h_model *m) {
    l2h_ctx *ctx = m->ctx;
    const l2h_config &c = m->c;
    m->flow = false;
    m->flow_why.clear();
    // automatic choice: this kernel where the model fits it (it is the fastest path), else one kernel per phase
    if (m->path_request != 3 && m->path_request != 0) return L2H_OK;
    const bool required = m->path_request == 3;
    FlowArgs a{};
    a.dim = c.dim;
    a.hidden = c.hidden_dim;
    a.hs = m->hs;
    a.n_heads = c.n_heads;
    a.n_kv_heads = c.n_kv_heads;
    a.kv_dim = m->kv_dim;
    a.seq_len = c.seq_len;
    a.n_layers = c.n_layers;
    a.vocab = c.vocab_size;
    a.neox = c.rope_is_neox;
    a.theta_scale = m->theta_scale;
    a.kv16 = m->kv16;
    std::vector<int> types;
    for (int l = 0; l < c.n_layers; l++)
        for (int r : {L2H_WQ, L2H_WK, L2H_WV, L2H_WO, L2H_W1, L2H_W2, L2H_W3}) types.push_back(m->L(l, r).type);
    const int grid = ctx->prop.multiProcessorCount;
    const int cls_type = m->glob[L2H_OUTPUT].type;
    std::string why;
    if (!k_flow_plan(a, types.data(), (int)types.size(), cls_type, grid, &why)) {
        m->flow_why = why;
        return required ? set_err(ctx, L2H_EINVAL, "streaming kernel not available: %s", why.c_str()) : L2H_OK;
    }
    if (m->L(0, L2H_RMS_ATT).layer_stride != m->L(0, L2H_RMS_FFN).layer_stride) {
        m->flow_why = "norm weight slabs differ";
        return required ? set_err(ctx, L2H_EINVAL, "streaming kernel not available: norm weight slabs differ") : L2H_OK;
    }
    if (!k_flow_fits(cls_type, grid, ctx->prop.multiProcessorCount, flow_form(a))) {
        m->flow_why = "its workgroups do not fit the device at once";
        return required ? set_err(ctx, L2H_EINVAL, "streaming kernel not available: its workgroups do not fit the device at once")
                        : L2H_OK;
    }
    if (a.f32) {  // fp32 model: no streams, the kernel reads the tensors where they lie
        const int roles[7] = {L2H_WQ, L2H_WK, L2H_WV, L2H_WO, L2H_W1, L2H_W3, L2H_W2};
        for (int i = 0; i < 7; i++) {
            a.f_w[i] = m->L(0, roles[i]).f32;
            a.f_stride[i] = m->L(0, roles[i]).layer_stride / 4;
        }
        a.f_w[7] = m->glob[L2H_OUTPUT].f32;
        a.f_stride[7] = 0;
    }
    std::vector<int64_t> off;
    int64_t total = 0;
    FlowTypedTables tt;
    FlowTypedDev typed;
    // tables that only the repack kernels read: freed on every way out of this function
    struct TmpTables {
        std::vector<void *> v;
        ~TmpTables() {
            for (void *p : v) (void)hipFree(p);
        }
    } tmp;
    int rc;
    if (a.mixed) {
        k_flow_typed_tables(a, types.data(), cls_type, grid, tt);
        off = tt.wave_off;
        total = tt.total;
        auto up = [&](const void *src, size_t bytes, const void **dst) -> int {
            void *v = nullptr;
            HIPCHK(ctx, hipMalloc(&v, std::max<size_t>(bytes, 16)));
            tmp.v.push_back(v);
            HIPCHK(ctx, hipMemcpy(v, src, bytes, hipMemcpyHostToDevice));
            *dst = v;
            return L2H_OK;
        };
        if ((rc = up(tt.piece_base.data(), tt.piece_base.size() * 8, (const void **)&typed.piece_base)) ||
            (rc = up(tt.cls_off.data(), tt.cls_off.size() * 8, (const void **)&typed.cls_off)) ||
            (rc = up(tt.piece_off.data(), tt.piece_off.size() * 8, (const void **)&typed.piece_off)) ||
            (rc = up(tt.piece_tag.data(), tt.piece_tag.size() * 2, (const void **)&typed.piece_tag)))
            return rc;
        unsigned int *wt = nullptr;
        if ((rc = dalloc(m, &wt, (int64_t)tt.wave_types.size(), false))) return rc;
        HIPCHK(ctx, hipMemcpy(wt, tt.wave_types.data(), tt.wave_types.size() * 4, hipMemcpyHostToDevice));
        a.wave_types = wt;
    } else if (!a.f32) {
        total = k_flow_offsets(a, cls_type, grid, off);
    }
    unsigned char *stream = nullptr;
    int64_t *off_dev = nullptr;
    if (!a.f32) {
        if ((rc = dalloc(m, &stream, total, false))) return rc;
        if ((rc = dalloc(m, &off_dev, (int64_t)off.size(), false))) return rc;
        HIPCHK(ctx, hipMemcpy(off_dev, off.data(), off.size() * 8, hipMemcpyHostToDevice));
    }
    for (int l = 0; l < c.n_layers && !a.f32; l++) {
        const DevTensor qkv[3] = {m->L(l, L2H_WQ), m->L(l, L2H_WK), m->L(l, L2H_WV)};
        const DevTensor wo[1] = {m->L(l, L2H_WO)};
        const DevTensor w13[2] = {m->L(l, L2H_W1), m->L(l, L2H_W3)};
        const DevTensor w2[1] = {m->L(l, L2H_W2)};
        HIPCHK(ctx, k_flow_repack(ctx->stream, a, stream, off_dev, 0, l, qkv, 3, grid, cls_type, typed));
        HIPCHK(ctx, k_flow_repack(ctx->stream, a, stream, off_dev, 1, l, wo, 1, grid, cls_type, typed));
        HIPCHK(ctx, k_flow_repack(ctx->stream, a, stream, off_dev, 2, l, w13, 2, grid, cls_type, typed));
        HIPCHK(ctx, k_flow_repack(ctx->stream, a, stream, off_dev, 3, l, w2, 1, grid, cls_type, typed));
    }
    if (!a.f32) HIPCHK(ctx, k_flow_repack(ctx->stream, a, stream, off_dev, 4, 0, &m->glob[L2H_OUTPUT], 1, grid, cls_type, typed));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    a.stream = stream;
    a.wave_off = off_dev;
    // the exchanged words live in uncached memory, zeroed like any other allocation
#define TA(p, n)                                                                                  \
    {                                                                                             \
        void *v_ = nullptr;                                                                       \
        const size_t b_ = (size_t)std::max<int64_t>((n), 1) * sizeof(*(p));                       \
        HIPCHK(ctx, uncached_alloc(ctx->device, b_, &v_));                                        \
        m->uc_allocs.push_back(v_);                                                               \
        HIPCHK(ctx, hipMemset(v_, 0, b_));                                                        \
        (p) = (decltype(p))v_;                                                                    \
    }
    TA(a.x_a, c.dim);
    TA(a.x_b, c.dim);
    TA(a.xo, 2 * (int64_t)c.dim);
    HIPCHK(ctx, hipMemset(a.x_a, 0xFF, (size_t)c.dim * 4));
    HIPCHK(ctx, hipMemset(a.x_b, 0xFF, (size_t)c.dim * 4));
    HIPCHK(ctx, hipMemset(a.xo, 0xFF, 2 * (size_t)c.dim * 4));
    TA(a.q, c.dim);
    TA(a.kcur, m->kv_dim);
    TA(a.vcur, m->kv_dim);
    TA(a.hbw, 2 * (int64_t)c.hidden_dim);
    HIPCHK(ctx, hipMemset(a.hbw, 0xFF, 2 * (size_t)c.hidden_dim * 4));
    TA(a.amax, 2 * grid);
    {
        const int64_t G = grid / c.n_heads;
        TA(a.att_x, (int64_t)c.n_heads * G * 3 + (int64_t)c.n_heads * G * m->hs * 2);
    }
    TA(a.abort_flag, 1);
    TA(a.tokw, 8 * 16);  // (eight copies, a 128-byte line each: FLOW_TOK_COPIES in k_flow.hip)
#undef TA
    a.kc = m->kc;
    a.vc = m->vc;
    a.logits = m->logits;
    a.rms_att = m->L(0, L2H_RMS_ATT).f32;
    a.rms_ffn = m->L(0, L2H_RMS_FFN).f32;
    a.rms_final = m->glob[L2H_RMS_FINAL].f32;
    a.norm_stride = m->L(0, L2H_RMS_ATT).layer_stride / 4;
    a.cache_layer_elems = m->cache_layer_elems;
    a.emb = m->glob[L2H_TOK_EMB];
    a.ctl = m->ctl;
    a.prompt = m->prompt_dev;
    a.out_tokens = m->out_tokens;
    a.max_out = m->max_out;
    a.spin_limit = 1u << 20;
#ifdef L2H_TIMELINE
    if ((rc = dalloc(m, &m->timeline, (int64_t)grid * 64 + 1024, true))) return rc;
    a.timeline = m->timeline;
#endif
    // several steps per launch where the cache is coherent between the steps (L2H_FLOW_STEPS: 1..64, for measurements)
    m->flow_steps_per_launch = m->kv_uncached ? 8 : 1;
    if (const char *e = getenv("L2H_FLOW_STEPS")) m->flow_steps_per_launch = std::min(64, std::max(1, atoi(e)));
    m->flow_args = a;
    m->flow_grid = grid;
    m->flow_cls_type = cls_type;
    m->flow_gen = 1;
    m->flow = true;
    return L2H_OK;
}

// The streaming kernel runs up to this many steps of the token loop per launch (the next step's token passes from
// workgroup 0 to the others inside the kernel): what lies between two launches, about 10 us, is paid once per that many tokens.
static hipError_t flow_launch_tokens(l2h_model *m, int n_tok) {
    if (g_flow_bound != m) {
        hipError_t eb = k_flow_bind(m->ctx->stream, m->flow_args);
        if (eb != hipSuccess) return eb;
        g_flow_bound = m;
    }
    hipError_t e = k_flow_launch(m->ctx->stream, m->flow_gen, n_tok, m->flow_cls_type, m->flow_grid, flow_form(m->flow_args));
    if (e == hipSuccess) m->flow_gen += (unsigned)n_tok * (5u * (unsigned)m->c.n_layers + 2u);
    return e;
}

static hipError_t mega_launch_token(l2h_model *m) {
    if (g_bound_model != m) {
        hipError_t e = k_mega_bind(m->ctx->stream, m->mega_ph);
        if (e != hipSuccess) return e;
        g_bound_model = m;
    }
    MegaArgs g = mega_args(m);
    hipError_t e = k_mega_launch(m->ctx->stream, g, m->mega_types[0], m->mega_types[1], m->mega_types[2],
                                 m->mega_types[3], m->mega_types[4], m->mega_grid, m->mega_lds);
    if (e == hipSuccess) m->bar_gen += 2ull + 5ull * (unsigned long long)m->c.n_layers;
    return e;
}

static hipError_t enqueue_token(l2h_model *m) {
    hipStream_t s = m->ctx->stream;
    const l2h_config &c = m->c;
    hipError_t e;
#define CK(call)                       \
    do {                               \
        e = (call);                    \
        if (e != hipSuccess) return e; \
    } while (0)
    // token embedding (:236) and this position's RoPE table
    CK(k_embed(s, m->glob[L2H_TOK_EMB], m->ctl, m->prompt_dev, m->x, m->rope_cs, m->hs, m->theta_scale));
    for (int l = 0; l < c.n_layers; l++) {
        float *kc = layer_kc(m, l), *vc = layer_vc(m, l);
        CK(launch_qkv(m, l));
        // attention (:263-278) -> xb: one launch while the sequence fits one workgroup's LDS, else split over time
        // (an fp16 cache is read by the split kernels only)
        if (c.seq_len <= 1024 && !m->kv16)
            CK(k_attention_fused(s, m->q, m->xb, kc, vc, m->ctl, m->hs, c.n_heads, c.n_kv_heads, c.seq_len));
        else
            CK(k_attention(s, m->qd, kc, vc, m->att, m->pd, m->part, m->xb, m->ctl, m->hs, c.n_heads, c.n_kv_heads,
                           c.seq_len, m->kv16));
        CK(launch_wo(m, l));
        CK(launch_w13(m, l));
        CK(launch_w2(m, l));
    }
    CK(launch_output(m));
    CK(k_argmax(s, m->logits, c.vocab_size, m->argmax_partial, m->ctl, m->out_tokens, m->max_out));  // :360
#undef CK
    return hipSuccess;
}

// Records the launch sequence of one token (launch path 1); positions and tokens are read from the
// control block on the device, so the recording is replayed unchanged for every step.
static int record_token(l2h_model *m) {
    l2h_ctx *ctx = m->ctx;
    if (m->exec || getenv("L2H_NO_GRAPH")) return L2H_OK;
    HIPCHK(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeGlobal));
    hipError_t e = enqueue_token(m);
    hipGraph_t g = nullptr;
    hipError_t e2 = hipStreamEndCapture(ctx->stream, &g);
    if (e != hipSuccess || e2 != hipSuccess) {
        if (g) (void)hipGraphDestroy(g);
        return set_err(ctx, L2H_EHIP, "recording the token launch sequence failed: %s",
                       hipGetErrorString(e != hipSuccess ? e : e2));
    }
    m->graph = g;
    HIPCHK(ctx, hipGraphInstantiate(&m->exec, m->graph, nullptr, nullptr, 0));
    return L2H_OK;
}

extern "C" int l2h_model_finalize(l2h_model *m) {
    if (!m) return L2H_EINVAL;
    l2h_ctx *ctx = m->ctx;
    if (m->finalized) return set_err(ctx, L2H_ESTATE, "model already finalized");
    const l2h_config &c = m->c;
    for (int r = 0; r < 3; r++)
        if (!m->glob[r].base) return set_err(ctx, L2H_ESTATE, "missing tensor %s", role_name(r));
    for (int l = 0; l < c.n_layers; l++)
        for (int r = 3; r < L2H_N_ROLES; r++)
            if (!m->L(l, r).base) return set_err(ctx, L2H_ESTATE, "missing blk.%d weights (%s)", l, role_name(r));
    HIPCHK(ctx, hipSetDevice(ctx->device));
    int rc;
    if ((rc = rehome_layers(m))) return rc;
#define DA(p, n, z)                       \
    if ((rc = dalloc(m, &(p), (n), (z)))) \
        return rc;
    DA(m->x, c.dim, true);
    DA(m->xb, c.dim, true);
    DA(m->xb2, c.dim, true);
    DA(m->hb, c.hidden_dim, true);
    DA(m->hb2, c.hidden_dim, true);
    DA(m->q, c.dim, true);
    DA(m->k, m->kv_dim, true);
    DA(m->v, m->kv_dim, true);
    DA(m->att, (int64_t)c.seq_len * c.n_heads, true);
    DA(m->logits, c.vocab_size, true);
    DA(m->qd, c.dim, true);
    DA(m->rope_cs, m->hs, true);
    DA(m->pd, (int64_t)c.seq_len * c.n_heads, true);
    const int ntiles = (c.seq_len + L2H_ATT_TILE - 1) / L2H_ATT_TILE;
    DA(m->part, (int64_t)ntiles * c.dim, true);
    m->cache_layer_elems = (int64_t)c.seq_len * m->kv_dim;
    if (m->kv16) {
        if (m->hs > 128 || m->hs % 32 != 0)
            return set_err(ctx, L2H_EINVAL, "an fp16 KV cache needs a head size that is a multiple of 32, at most 128");
        if (m->path_request == 2) return set_err(ctx, L2H_EINVAL, "an fp16 KV cache does not run on launch path 2");
    }
    // (an fp16 cache takes half the floats)
    // A launch of the streaming kernel that runs several steps of the token loop reads, in a later step, cache rows that
    // another XCD's workgroups appended in an earlier one: rows in ordinary memory would still sit in the writer's L2
    // (and stale lines in the reader's), which only the end of a kernel puts right.  Where no two heads share a cache
    // row (n_kv_heads == n_heads: nothing is read twice, the L2 holds nothing worth keeping) the cache therefore lives
    // in uncached memory, and such a model decodes several steps per launch; with shared rows it stays in ordinary memory
    // and every step is a launch.
    {
        const char *env = getenv("L2H_KV_UNCACHED");
        m->kv_uncached = env ? atoi(env) != 0 : (c.n_heads == c.n_kv_heads && (m->path_request == 0 || m->path_request == 3));
        const int64_t n = m->cache_layer_elems * c.n_layers / (m->kv16 ? 2 : 1) + 1;
        if (m->kv_uncached) {
            for (float **p : {&m->kc, &m->vc}) {
                void *v = nullptr;
                HIPCHK(ctx, uncached_alloc(ctx->device, (size_t)n * 4, &v));
                m->uc_allocs.push_back(v);
                HIPCHK(ctx, hipMemset(v, 0, (size_t)n * 4));
                *p = (float *)v;
            }
        } else {
            DA(m->kc, n, true);
            DA(m->vc, n, true);
        }
    }
    DA(m->ctl, 1, true);
    DA(m->prompt_dev, c.seq_len, true);
    m->max_out = c.seq_len;
    DA(m->out_tokens, m->max_out, true);
    DA(m->argmax_partial, std::max(L2H_ARGMAX_BLOCKS, ctx->prop.multiProcessorCount), true);
#undef DA
    HIPCHK(ctx, hipDeviceSynchronize());
    if ((rc = mega_setup(m))) return rc;
    if ((rc = flow_setup(m))) return rc;

    if (!m->mega && !m->flow && (rc = record_token(m))) return rc;
    m->finalized = true;
    return L2H_OK;
}

static int run_steps(l2h_model *m, int n) {
    l2h_ctx *ctx = m->ctx;
    for (int i = 0; i < n; i++) {
        if (m->flow) {
            const int n_tok = std::min(n - i, m->flow_steps_per_launch);
            hipError_t e = flow_launch_tokens(m, n_tok);
            if (e != hipSuccess) return set_err(ctx, L2H_EHIP, "decode kernel launch failed: %s", hipGetErrorString(e));
            i += n_tok - 1;
        } else if (m->mega) {
            hipError_t e = mega_launch_token(m);
            if (e != hipSuccess) return set_err(ctx, L2H_EHIP, "decode kernel launch failed: %s", hipGetErrorString(e));
        } else if (m->exec) {
            HIPCHK(ctx, hipGraphLaunch(m->exec, ctx->stream));
        } else {
            hipError_t e = enqueue_token(m);
            if (e != hipSuccess) return set_err(ctx, L2H_EHIP, "token launch failed: %s", hipGetErrorString(e));
        }
    }
    return L2H_OK;
}

// after the stream has drained: did a workgroup of the persistent kernel give up at a barrier?
static int mega_check(l2h_model *m) {
    if (m->flow) {
        unsigned int ab = 0;
        HIPCHK(m->ctx, hipMemcpy(&ab, m->flow_args.abort_flag, 4, hipMemcpyDeviceToHost));
        if (!ab) return L2H_OK;
        HIPCHK(m->ctx, hipMemset(m->flow_args.abort_flag, 0, 4));
        // all words "not written"
        HIPCHK(m->ctx, hipMemset(m->flow_args.hbw, 0xFF, 2 * (size_t)m->c.hidden_dim * 4));
        HIPCHK(m->ctx, hipMemset(m->flow_args.x_a, 0xFF, (size_t)m->c.dim * 4));
        HIPCHK(m->ctx, hipMemset(m->flow_args.x_b, 0xFF, (size_t)m->c.dim * 4));
        HIPCHK(m->ctx, hipMemset(m->flow_args.xo, 0xFF, 2 * (size_t)m->c.dim * 4));
        // Where the library chose this path itself, the following calls run one kernel per phase: a launch whose
        // workgroups are not all resident at once (another process on the GPU) would give up at every token.  A
        // caller that asked for path 3 keeps it.
        if (m->path_request == 0) {
            const int rc = record_token(m);
            if (rc == L2H_OK) {
                m->flow = false;
                m->flow_why = "a wait of the streaming kernel ran into its limit (are its workgroups resident at once?); "
                              "the model now runs one kernel per phase";
                if (g_flow_bound == m) g_flow_bound = nullptr;
                return set_err(m->ctx, L2H_EHIP, "streaming decode kernel: a wait for activations timed out; the model "
                                                 "runs on launch path 1 from now on");
            }
        }
        return set_err(m->ctx, L2H_EHIP, "streaming decode kernel: a wait for activations timed out");
    }
    if (!m->mega) return L2H_OK;
    unsigned int ab = 0;
    HIPCHK(m->ctx, hipMemcpy(&ab, &m->bar->abort, 4, hipMemcpyDeviceToHost));
    if (!ab) return L2H_OK;
    HIPCHK(m->ctx, hipMemset(m->bar, 0, sizeof(GridBar)));
    m->bar_gen = 0;
    return set_err(m->ctx, L2H_EHIP, "persistent decode kernel: a grid barrier timed out (workgroups not co-resident?)");
}

extern "C" int l2h_state_reset(l2h_model *m) {
    if (!m) return L2H_EINVAL;
    if (!m->finalized) return set_err(m->ctx, L2H_ESTATE, "model not finalized");
    const size_t bytes = (size_t)m->cache_layer_elems * m->c.n_layers * (m->kv16 ? 2 : 4);
    HIPCHK(m->ctx, hipMemsetAsync(m->kc, 0, bytes, m->ctx->stream));
    HIPCHK(m->ctx, hipMemsetAsync(m->vc, 0, bytes, m->ctx->stream));
    HIPCHK(m->ctx, hipStreamSynchronize(m->ctx->stream));
    return L2H_OK;
}

static int kv_xfer(l2h_model *m, int layer, int pos0, int n, float *k, float *v, bool to_cache) {
    if (!m) return L2H_EINVAL;
    l2h_ctx *ctx = m->ctx;
    if (!m->finalized) return set_err(ctx, L2H_ESTATE, "model not finalized");
    if (layer < 0 || layer >= m->c.n_layers || pos0 < 0 || n < 0 || pos0 + n > m->c.seq_len || !k || !v)
        return set_err(ctx, L2H_EINVAL, "kv range out of bounds (layer %d, pos %d, n %d)", layer, pos0, n);
    if (n == 0) return L2H_OK;
    const size_t bytes = (size_t)n * m->kv_dim * 4;
    float *dk = nullptr, *dv = nullptr;
    HIPCHK(ctx, hipMalloc((void **)&dk, bytes));
    hipError_t e = hipMalloc((void **)&dv, bytes);
    if (e == hipSuccess && to_cache) {
        e = hipMemcpy(dk, k, bytes, hipMemcpyHostToDevice);
        if (e == hipSuccess) e = hipMemcpy(dv, v, bytes, hipMemcpyHostToDevice);
    }
    if (e == hipSuccess)
        e = k_kv_layout(ctx->stream, layer_kc(m, layer), layer_vc(m, layer), dk, dv, pos0, n, m->hs, m->c.n_kv_heads,
                        m->c.seq_len, to_cache, m->kv16);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess && !to_cache) {
        e = hipMemcpy(k, dk, bytes, hipMemcpyDeviceToHost);
        if (e == hipSuccess) e = hipMemcpy(v, dv, bytes, hipMemcpyDeviceToHost);
    }
    (void)hipFree(dk);
    if (dv) (void)hipFree(dv);
    if (e != hipSuccess) return set_err(ctx, L2H_EHIP, "kv transfer failed: %s", hipGetErrorString(e));
    return L2H_OK;
}

extern "C" int l2h_kv_write(l2h_model *m, int layer, int pos0, int n, const float *k, const float *v) {
    return kv_xfer(m, layer, pos0, n, (float *)k, (float *)v, true);
}
extern "C" int l2h_kv_read(l2h_model *m, int layer, int pos0, int n, float *k, float *v) {
    return kv_xfer(m, layer, pos0, n, k, v, false);
}

static int generate_impl(l2h_model *m, const int32_t *prompt, int n_prompt, int pos0, int n_new, int32_t *out,
                         float *last_logits, float *decode_ms) {
    if (!m) return L2H_EINVAL;
    l2h_ctx *ctx = m->ctx;
    if (!m->finalized) return set_err(ctx, L2H_ESTATE, "model not finalized");
    if (!prompt || n_prompt < 1) return set_err(ctx, L2H_EINVAL, "prompt cannot be empty");  // inference.jl:326-328
    if (n_new < 0 || pos0 < 0) return set_err(ctx, L2H_EINVAL, "negative count");
    if (n_prompt > m->c.seq_len) return set_err(ctx, L2H_EINVAL, "prompt of %d tokens exceeds seq_len %d", n_prompt, m->c.seq_len);
    const int total = n_prompt - 1 + n_new;
    if (pos0 + total > m->c.seq_len)
        return set_err(ctx, L2H_EINVAL, "pos0 %d + %d steps exceeds seq_len %d", pos0, total, m->c.seq_len);
    if (n_new > 0 && !out) return set_err(ctx, L2H_EINVAL, "out is NULL");
    for (int i = 0; i < n_prompt; i++)
        if (prompt[i] < 0 || prompt[i] >= m->c.vocab_size)
            return set_err(ctx, L2H_EINVAL, "prompt[%d] = %d outside vocabulary", i, prompt[i]);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DecodeCtl h{};
    h.token = prompt[0];
    h.pos = pos0;
    h.step = 0;
    h.n_prompt = n_prompt;
    h.last_argmax = 0;
    h.n_out = 0;
    HIPCHK(ctx, hipMemcpyAsync(m->prompt_dev, prompt, (size_t)n_prompt * 4, hipMemcpyHostToDevice, ctx->stream));
    HIPCHK(ctx, hipMemcpyAsync(m->ctl, &h, sizeof h, hipMemcpyHostToDevice, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    int rc;
    if (decode_ms) {
        hipEvent_t e0 = nullptr, e1 = nullptr;
        HIPCHK(ctx, hipEventCreate(&e0));
        hipError_t he = hipEventCreate(&e1);
        rc = L2H_OK;
        if (he == hipSuccess) rc = run_steps(m, total - n_new);
        if (he == hipSuccess && rc == L2H_OK) he = hipEventRecord(e0, ctx->stream);
        if (he == hipSuccess && rc == L2H_OK) rc = run_steps(m, n_new);
        if (he == hipSuccess && rc == L2H_OK) he = hipEventRecord(e1, ctx->stream);
        if (he == hipSuccess && rc == L2H_OK) he = hipEventSynchronize(e1);
        if (he == hipSuccess && rc == L2H_OK) he = hipEventElapsedTime(decode_ms, e0, e1);
        (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        if (rc) return rc;
        if (he != hipSuccess) return set_err(ctx, L2H_EHIP, "timing the decode steps failed: %s", hipGetErrorString(he));
    } else {
        if ((rc = run_steps(m, total))) return rc;
    }
    if (n_new > 0)
        HIPCHK(ctx, hipMemcpyAsync(out, m->out_tokens, (size_t)n_new * 4, hipMemcpyDeviceToHost, ctx->stream));
    if (last_logits)
        HIPCHK(ctx, hipMemcpyAsync(last_logits, m->logits, (size_t)m->c.vocab_size * 4, hipMemcpyDeviceToHost,
                                   ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return mega_check(m);
}

// ---- batched prompt pass --------------------------------------------------------------------
#define L2H_PREFILL_CHUNK 2048

static int prefill_buffers(l2h_model *m, int cap) {
    if (m->pf_cap >= cap) return L2H_OK;
    const l2h_config &c = m->c;
    int rc;
    // earlier, smaller buffers stay in the allocation list and are released with the model
#define DA(p, n)                            \
    if ((rc = dalloc(m, &(p), (n), false))) \
        return rc;
    DA(m->pf_x, (int64_t)cap * c.dim);
    DA(m->pf_raw, (int64_t)cap * (c.dim + 2 * m->kv_dim));
    DA(m->pf_cs, (int64_t)cap * m->hs);
    DA(m->pf_xn, (int64_t)cap * c.dim);
    DA(m->pf_q, (int64_t)cap * c.dim);
    DA(m->pf_att, (int64_t)cap * c.dim);
    DA(m->pf_hb, (int64_t)cap * c.hidden_dim);
    DA(m->pf_tok, cap);
    m->pf_kvt_tiles = (c.seq_len + 31) / 32;
    DA(m->pf_kvt, (int64_t)c.n_kv_heads * m->pf_kvt_tiles * k_pf_kv_tile_bytes(m->hs));
#undef DA
    m->pf_cap = cap;
    return L2H_OK;
}

// Expands every layer matrix to bf16 once (the values the fused product kernel would form in LDS), so
// that later prompt passes run plain bf16 products.  2 bytes per weight stay resident; when that does
// not fit beside 2 GiB of head room, or dim or hidden_dim is not a multiple of 64, the fused kernels
// stay in use.
// (re)writes the copy: w1 | w3 always as the product kernel's tiles, the three plain products' matrices as tiles or as
// plain rows
static int prefill_expand(l2h_model *m, bool plain) {
    const l2h_config &c = m->c;
    const int64_t dim = c.dim, kvd = m->kv_dim, hid = c.hidden_dim;
    hipStream_t s = m->ctx->stream;
    const int pl = plain ? 1 : 0;
    for (int l = 0; l < c.n_layers; l++) {
        uint16_t *base = m->pf_wbf + (int64_t)l * m->pf_wbf_layer;
        const DevTensor w[3] = {m->L(l, L2H_WQ), m->L(l, L2H_WK), m->L(l, L2H_WV)};
        const int64_t row0[3] = {0, dim, dim + kvd};
        for (int i = 0; i < 3; i++) HIPCHK(m->ctx, k_pf_expand(s, w + i, 1, 0, dim, base, row0[i], i == 2, pl));
        const DevTensor wo = m->L(l, L2H_WO), w2 = m->L(l, L2H_W2);
        const DevTensor w13[2] = {m->L(l, L2H_W1), m->L(l, L2H_W3)};
        HIPCHK(m->ctx, k_pf_expand(s, &wo, 1, 0, dim, base + m->pf_off_wo, 0, 1, pl));
        HIPCHK(m->ctx, k_pf_expand(s, w13, 2, 1, dim, base + m->pf_off_w13, 0, 1, 0));
        HIPCHK(m->ctx, k_pf_expand(s, &w2, 1, 0, hid, base + m->pf_off_w2, 0, 1, pl));
    }
    HIPCHK(m->ctx, hipStreamSynchronize(s));
    m->pf_plain = plain;
    return L2H_OK;
}

static int prefill_weights(l2h_model *m) {
    // the library for the plain products: opened once; L2H_PF_LIBRARY=0 keeps every product in this library's kernels
    const char *env = getenv("L2H_PF_LIBRARY");
    const bool want = m->pf_library_mode != 0 && !(env && atoi(env) == 0);
    if (want && !m->pf_lt_tried) {
        m->pf_lt_tried = true;
        m->pf_lt = pf_lt_open(&m->pf_lt_why);
    }
    const bool plain = want && m->pf_lt != nullptr;
    if (m->pf_copy_tried) {
        if (m->pf_wbf && plain != m->pf_plain) return prefill_expand(m, plain);
        return L2H_OK;
    }
    m->pf_copy_tried = true;
    const l2h_config &c = m->c;
    const int64_t dim = c.dim, kvd = m->kv_dim, hid = c.hidden_dim;
    if (dim % 64 != 0 || hid % 64 != 0) return L2H_OK;
    auto pad_rows = [](int64_t r) { return (r + 255) / 256 * 256; };  // whole tiles of 256 rows
    m->pf_off_wo = pad_rows(dim + 2 * kvd) * dim;
    m->pf_off_w13 = m->pf_off_wo + pad_rows(dim) * dim;
    m->pf_off_w2 = m->pf_off_w13 + pad_rows(2 * hid) * dim;
    m->pf_wbf_layer = m->pf_off_w2 + pad_rows(dim) * hid;
    const size_t bytes = (size_t)m->pf_wbf_layer * c.n_layers * 2;
    size_t free_b = 0, total_b = 0;
    HIPCHK(m->ctx, hipMemGetInfo(&free_b, &total_b));
    if (free_b < bytes + ((size_t)2 << 30)) return L2H_OK;
    uint16_t *buf = nullptr;
    int rc;
    if ((rc = dalloc(m, &buf, (int64_t)(bytes / 2), false))) return rc;
    m->pf_wbf = buf;
    if ((rc = prefill_expand(m, plain))) {
        m->pf_wbf = nullptr;
        return rc;
    }
    return L2H_OK;
}

static hipError_t prefill_chunk(l2h_model *m, int M, int pos0) {
    hipStream_t s = m->ctx->stream;
    const l2h_config &c = m->c;
    const int dim = c.dim, kvd = m->kv_dim;
    hipError_t e;
#define CK(call)                       \
    do {                               \
        e = (call);                    \
        if (e != hipSuccess) return e; \
    } while (0)
    CK(k_pf_embed(s, m->glob[L2H_TOK_EMB], m->pf_tok, m->pf_x, M));
    CK(k_pf_rope_table(s, m->pf_cs, pos0, M, m->hs / 2, m->theta_scale));
    for (int l = 0; l < c.n_layers; l++) {
        float *kc = m->kc + (int64_t)l * m->cache_layer_elems;
        float *vc = m->vc + (int64_t)l * m->cache_layer_elems;
        CK(k_pf_rmsnorm(s, m->pf_x, m->L(l, L2H_RMS_ATT).f32, m->pf_xn, M, dim));
        const uint16_t *wb = (m->pf_wbf && m->pf_copy_mode) ? m->pf_wbf + (int64_t)l * m->pf_wbf_layer : nullptr;
        const bool lib = wb && m->pf_plain;  // (plain rows in the copy: the plain products go through hipBLASLt)
        if (lib) {
            CK(pf_lt_gemm(m->pf_lt, s, wb, m->pf_xn, m->pf_raw, M, dim + 2 * kvd, dim, dim + 2 * kvd, false, &m->pf_lt_err));
        } else if (wb) {
            CK(k_pf_gemm(s, nullptr, 0, 0, wb, dim + 2 * kvd, m->pf_xn, M, dim, PF_STORE, m->pf_raw, dim + 2 * kvd, 0,
                         nullptr, 0));
        } else {
            // q | k | v columns of pf_raw; consecutive tensors of one type share a launch
            const DevTensor w[3] = {m->L(l, L2H_WQ), m->L(l, L2H_WK), m->L(l, L2H_WV)};
            const int64_t col[3] = {0, dim, dim + kvd};
            for (int i = 0; i < 3;) {
                int j = i + 1;
                while (j < 3 && w[j].type == w[i].type) j++;
                CK(k_pf_gemm(s, w + i, j - i, 0, nullptr, 0, m->pf_xn, M, dim, PF_STORE, m->pf_raw, dim + 2 * kvd,
                             col[i], nullptr, 0));
                i = j;
            }
        }
        CK(k_pf_rope_scatter(s, m->pf_raw, m->pf_cs, m->pf_q, kc, vc, M, pos0, dim, kvd, m->hs, c.seq_len,
                             c.rope_is_neox));
        CK(k_pf_kv_tiles(s, kc, vc, m->pf_kvt, (pos0 + M + 31) / 32, m->pf_kvt_tiles, m->hs, c.n_kv_heads, c.seq_len));
        CK(k_pf_attention(s, m->pf_q, m->pf_att, m->pf_kvt, m->pf_kvt_tiles, M, pos0, m->hs, c.n_heads, c.n_kv_heads, dim));
        const DevTensor wo = m->L(l, L2H_WO);
        if (lib)
            CK(pf_lt_gemm(m->pf_lt, s, wb + m->pf_off_wo, m->pf_att, m->pf_x, M, dim, dim, dim, true, &m->pf_lt_err));
        else
            CK(k_pf_gemm(s, &wo, 1, 0, wb ? wb + m->pf_off_wo : nullptr, dim, m->pf_att, M, dim, PF_RESID, m->pf_x, dim, 0,
                         nullptr, 0));
        CK(k_pf_rmsnorm(s, m->pf_x, m->L(l, L2H_RMS_FFN).f32, m->pf_xn, M, dim));
        const DevTensor w13[2] = {m->L(l, L2H_W1), m->L(l, L2H_W3)};
        CK(k_pf_gemm(s, w13, 2, 1, wb ? wb + m->pf_off_w13 : nullptr, 2 * (int64_t)c.hidden_dim, m->pf_xn, M, dim,
                     PF_SWIGLU, nullptr, 0, 0, m->pf_hb, c.hidden_dim));
        const DevTensor w2 = m->L(l, L2H_W2);
        if (lib)
            CK(pf_lt_gemm(m->pf_lt, s, wb + m->pf_off_w2, m->pf_hb, m->pf_x, M, dim, c.hidden_dim, dim, true, &m->pf_lt_err));
        else
            CK(k_pf_gemm(s, &w2, 1, 0, wb ? wb + m->pf_off_w2 : nullptr, dim, m->pf_hb, M, c.hidden_dim, PF_RESID, m->pf_x,
                         dim, 0, nullptr, 0));
    }
#undef CK
    return hipSuccess;
}

extern "C" int l2h_prefill(l2h_model *m, const int32_t *tokens, int n, int pos0, float *last_logits,
                           int32_t *next_token) {
    if (!m) return L2H_EINVAL;
    l2h_ctx *ctx = m->ctx;
    if (!m->finalized) return set_err(ctx, L2H_ESTATE, "model not finalized");
    if (!tokens || n < 1) return set_err(ctx, L2H_EINVAL, "prompt cannot be empty");
    if (pos0 < 0 || pos0 + n > m->c.seq_len)
        return set_err(ctx, L2H_EINVAL, "positions %d..%d outside the cache of %d", pos0, pos0 + n - 1, m->c.seq_len);
    for (int i = 0; i < n; i++)
        if (tokens[i] < 0 || tokens[i] >= m->c.vocab_size)
            return set_err(ctx, L2H_EINVAL, "tokens[%d] = %d outside vocabulary", i, tokens[i]);
    if (m->kv16) return set_err(ctx, L2H_ESTATE, "the batched prompt pass writes an fp32 cache only (this model's is fp16)");
    if (!k_pf_attention_supported(m->hs))
        return set_err(ctx, L2H_EINVAL, "batched prompt pass needs a head size of 32, 64, 96 or 128 (have %d)", m->hs);
    if (m->c.dim % 8 != 0 || m->c.hidden_dim % 8 != 0)
        return set_err(ctx, L2H_EINVAL, "batched prompt pass needs dim and hidden_dim to be multiples of 8");
    for (int l = 0; l < m->c.n_layers; l++)
        if (m->L(l, L2H_W1).type != m->L(l, L2H_W3).type)
            return set_err(ctx, L2H_EINVAL, "batched prompt pass needs w1 and w3 of one type (layer %d)", l);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    int rc;
    if ((rc = prefill_buffers(m, std::min(n, L2H_PREFILL_CHUNK)))) return rc;
    if (m->pf_copy_mode && (rc = prefill_weights(m))) return rc;
    int M = 0;
    for (int c0 = 0; c0 < n; c0 += M) {
        M = std::min(m->pf_cap, n - c0);
        if (m->pf_wbf && m->pf_copy_mode && m->pf_plain) {
            // The library must have an algorithm for this chunk's three products before anything is computed with it
            // (it may be installed without the kernels for this device): where it has none, the own kernels take over
            // for good and the copy's matrices go back to tiles.
            const int64_t dim = m->c.dim, kvd = m->kv_dim, hid = m->c.hidden_dim;
            const uint16_t *wb = m->pf_wbf;
            const bool ok =
                pf_lt_gemm(m->pf_lt, ctx->stream, wb, m->pf_xn, nullptr, M, dim + 2 * kvd, dim, dim + 2 * kvd, false, &m->pf_lt_err) == hipSuccess &&
                pf_lt_gemm(m->pf_lt, ctx->stream, wb + m->pf_off_wo, m->pf_att, nullptr, M, dim, dim, dim, true, &m->pf_lt_err) == hipSuccess &&
                pf_lt_gemm(m->pf_lt, ctx->stream, wb + m->pf_off_w2, m->pf_hb, nullptr, M, dim, hid, dim, true, &m->pf_lt_err) == hipSuccess;
            if (!ok) {
                (void)hipGetLastError();
                m->pf_lt_why = "hipBLASLt has no algorithm for the prompt pass's products: " + m->pf_lt_err;
                m->pf_lt_err.clear();
                pf_lt_close(m->pf_lt);
                m->pf_lt = nullptr;
                if ((rc = prefill_expand(m, false))) return rc;
            }
        }
        HIPCHK(ctx, hipMemcpyAsync(m->pf_tok, tokens + c0, (size_t)M * 4, hipMemcpyHostToDevice, ctx->stream));
        hipError_t e = prefill_chunk(m, M, pos0 + c0);
        if (e != hipSuccess)
            return set_err(ctx, L2H_EHIP, "prompt pass launch failed: %s%s%s", hipGetErrorString(e),
                           m->pf_lt_err.empty() ? "" : "; ", m->pf_lt_err.c_str());
    }
    // last position: its hidden state becomes the decode state; classifier and argmax as in a decode step
    HIPCHK(ctx, hipMemcpyAsync(m->x, m->pf_x + (int64_t)(M - 1) * m->c.dim, (size_t)m->c.dim * 4,
                               hipMemcpyDeviceToDevice, ctx->stream));
    DecodeCtl h{};
    h.token = tokens[n - 1];
    h.pos = pos0 + n - 1;
    h.n_prompt = 1;
    HIPCHK(ctx, hipMemcpyAsync(m->ctl, &h, sizeof h, hipMemcpyHostToDevice, ctx->stream));
    hipError_t e = launch_output(m);
    if (e == hipSuccess)
        e = k_argmax(ctx->stream, m->logits, m->c.vocab_size, m->argmax_partial, m->ctl, m->out_tokens, m->max_out);
    if (e != hipSuccess) return set_err(ctx, L2H_EHIP, "classifier launch failed: %s", hipGetErrorString(e));
    if (next_token)
        HIPCHK(ctx, hipMemcpyAsync(next_token, m->out_tokens, 4, hipMemcpyDeviceToHost, ctx->stream));
    if (last_logits)
        HIPCHK(ctx, hipMemcpyAsync(last_logits, m->logits, (size_t)m->c.vocab_size * 4, hipMemcpyDeviceToHost,
                                   ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return L2H_OK;
}

extern "C" int l2h_generate_greedy(l2h_model *m, const int32_t *prompt, int n_prompt, int pos0, int n_new,
                                   int32_t *out, float *last_logits) {
    return generate_impl(m, prompt, n_prompt, pos0, n_new, out, last_logits, nullptr);
}

extern "C" int l2h_generate_greedy_timed(l2h_model *m, const int32_t *prompt, int n_prompt, int pos0, int n_new,
                                         int32_t *out, float *decode_ms) {
    if (!decode_ms) return set_err(m ? m->ctx : nullptr, L2H_EINVAL, "decode_ms is NULL");
    return generate_impl(m, prompt, n_prompt, pos0, n_new, out, nullptr, decode_ms);
}

extern "C" int l2h_forward(l2h_model *m, int token, int pos, float *logits, int32_t *argmax) {
    int32_t tok = token, next = 0;
    int rc = generate_impl(m, &tok, 1, pos, 1, &next, logits, nullptr);
    if (rc == L2H_OK && argmax) *argmax = next;
    return rc;
}

extern "C" int l2h_sample(l2h_model *m, float temperature, float u, int32_t *token, float *probs) {
    if (!m || !token) return set_err(m ? m->ctx : nullptr, L2H_EINVAL, "l2h_sample: NULL argument");
    l2h_ctx *ctx = m->ctx;
    if (!m->finalized) return set_err(ctx, L2H_ESTATE, "model not finalized");
    if (!(temperature > 0.0f) || !(u >= 0.0f && u < 1.0f))
        return set_err(ctx, L2H_EINVAL, "need temperature > 0 and 0 <= u < 1 (got %g, %g)", (double)temperature, (double)u);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    if (!m->sample_p) {
        int rc;
        if ((rc = dalloc(m, &m->sample_p, m->c.vocab_size, false))) return rc;
        if ((rc = dalloc(m, &m->sample_out, 1, true))) return rc;
    }
    HIPCHK(ctx, k_sample(ctx->stream, m->logits, m->c.vocab_size, temperature, u, m->sample_p, m->sample_out));
    HIPCHK(ctx, hipMemcpyAsync(token, m->sample_out, 4, hipMemcpyDeviceToHost, ctx->stream));
    if (probs)
        HIPCHK(ctx, hipMemcpyAsync(probs, m->sample_p, (size_t)m->c.vocab_size * 4, hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return L2H_OK;
}

extern "C" int l2h_state_read(l2h_model *m, int which, float *host, int64_t n) {
    if (!m || !host) return L2H_EINVAL;
    if (!m->finalized) return set_err(m->ctx, L2H_ESTATE, "model not finalized");
    const float *src = nullptr;
    int64_t len = 0;
    switch (which) {
    case 0: src = m->x; len = m->c.dim; break;
    case 1: src = m->xb; len = m->c.dim; break;
    case 2: src = m->q; len = m->c.dim; break;
    case 5: src = m->hb; len = m->c.hidden_dim; break;
    case 6: src = m->logits; len = m->c.vocab_size; break;
    default: return set_err(m->ctx, L2H_EINVAL, "unknown state buffer %d", which);
    }
    if (n != len) return set_err(m->ctx, L2H_EINVAL, "buffer %d holds %lld floats, asked for %lld", which,
                                 (long long)len, (long long)n);
    HIPCHK(m->ctx, hipStreamSynchronize(m->ctx->stream));
    HIPCHK(m->ctx, hipMemcpy(host, src, (size_t)len * 4, hipMemcpyDeviceToHost));
    return L2H_OK;
}

// ------------------------------------------------------------------------------------------
// single operators: upload, run the same kernel the model path uses, download
// ------------------------------------------------------------------------------------------
struct DevBuf {  // frees on scope exit
    void *p = nullptr;
    ~DevBuf() {
        if (p) (void)hipFree(p);
    }
    hipError_t alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 1); }
    template <class T>
    T *as() { return (T *)p; }
};

static int q8_pack_blocks(l2h_ctx *ctx, const Q8Dev &q, int64_t n, void *out_blocks) {
    const int64_t nb = n / QK_K;
    std::vector<int8_t> qs((size_t)n);
    std::vector<int16_t> bs((size_t)n / 16);
    std::vector<float> d((size_t)nb);
    HIPCHK(ctx, hipMemcpy(qs.data(), q.qs, (size_t)n, hipMemcpyDeviceToHost));
    HIPCHK(ctx, hipMemcpy(bs.data(), q.bsums, (size_t)n / 8, hipMemcpyDeviceToHost));
    HIPCHK(ctx, hipMemcpy(d.data(), q.d, (size_t)nb * 4, hipMemcpyDeviceToHost));
    char *o = (char *)out_blocks;
    for (int64_t b = 0; b < nb; b++, o += 292) {  // block_q8_K: f32 d, i8 qs[256], i16 bsums[16]
        memcpy(o, &d[b], 4);
        memcpy(o + 4, &qs[b * 256], 256);
        memcpy(o + 260, &bs[b * 16], 32);
    }
    return L2H_OK;
}

extern "C" int l2h_quantize_q8k(l2h_ctx *ctx, const float *x, int64_t n, void *out_blocks) {
    if (!ctx || !x || !out_blocks) return set_err(ctx, L2H_EINVAL, "l2h_quantize_q8k: NULL argument");
    if (n < 0 || n % QK_K != 0) return set_err(ctx, L2H_EINVAL, "n = %lld is not a multiple of 256", (long long)n);
    if (n == 0) return L2H_OK;
    // the rule's "first element of largest magnitude" has no meaning for a NaN, and an infinite extreme gives a scale of 0
    for (int64_t i = 0; i < n; i++)
        if (!std::isfinite(x[i])) return set_err(ctx, L2H_EINVAL, "x[%lld] is not finite", (long long)i);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevBuf dx;
    HIPCHK(ctx, dx.alloc((size_t)n * 4));
    HIPCHK(ctx, hipMemcpy(dx.p, x, (size_t)n * 4, hipMemcpyHostToDevice));
    Q8Dev q;
    std::vector<void *> tr;
    int rc = q8_alloc(ctx, n, &q, &tr);
    if (rc) return rc;
    // The library has two forms of this quantizer: a block per wavefront (the per-phase kernels' prologue) and four
    // blocks per wavefront (the streaming kernel's staging).  Both run here and must agree byte for byte.
    Q8Dev q2;
    std::vector<void *> tr2;
    rc = q8_alloc(ctx, n, &q2, &tr2);
    if (rc) {
        (void)hipFree(tr[0]);
        return rc;
    }
    hipError_t e = k_stage_dump(ctx->stream, dx.as<float>(), nullptr, n, PRO_QUANT, q, nullptr);
    if (e == hipSuccess) e = k_quantize_rows16(ctx->stream, dx.as<float>(), n, q2);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) {
        const size_t bytes = (size_t)(n / QK_K) * 292;
        std::vector<unsigned char> other(bytes);
        rc = q8_pack_blocks(ctx, q, n, out_blocks);
        if (rc == L2H_OK) rc = q8_pack_blocks(ctx, q2, n, other.data());
        if (rc == L2H_OK && memcmp(other.data(), out_blocks, bytes) != 0)
            rc = set_err(ctx, L2H_EHIP, "the two forms of the q8_K quantizer disagree");
    } else {
        rc = set_err(ctx, L2H_EHIP, "quantize failed: %s", hipGetErrorString(e));
    }
    (void)hipFree(tr[0]);
    (void)hipFree(tr2[0]);
    return rc;
}

extern "C" int l2h_dequantize(l2h_ctx *ctx, int type, const void *blocks, int64_t nb, float *y) {
    if (!ctx || !blocks || !y) return set_err(ctx, L2H_EINVAL, "l2h_dequantize: NULL argument");
    if (!type_ok(type)) return set_err(ctx, L2H_ETYPE, "tensor type %d not implemented", type);
    if (nb < 0) return set_err(ctx, L2H_EINVAL, "negative block count");
    if (nb == 0) return L2H_OK;
    HIPCHK(ctx, hipSetDevice(ctx->device));
    const int64_t ne0 = type == L2H_TYPE_F32 ? nb : nb * QK_K;
    DevTensor t;
    int rc = dev_tensor_alloc(ctx, type, ne0, 1, &t);
    if (rc) return rc;
    rc = dev_tensor_upload(ctx, &t, blocks);
    if (rc == L2H_OK) {
        DevBuf dy;
        hipError_t e = dy.alloc((size_t)ne0 * 4);
        if (e == hipSuccess) e = k_dequant(ctx->stream, t, 0, 1, dy.as<float>());
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e == hipSuccess) e = hipMemcpy(y, dy.p, (size_t)ne0 * 4, hipMemcpyDeviceToHost);
        if (e != hipSuccess) rc = set_err(ctx, L2H_EHIP, "dequantize failed: %s", hipGetErrorString(e));
    }
    dev_tensor_free(&t);
    return rc;
}

extern "C" int l2h_matmul(l2h_ctx *ctx, int type, const void *A, int64_t ne0, int64_t ne1, const float *x, float *y,
                          int32_t *I_sc, int32_t *I_min) {
    if (!ctx || !A || !x || !y) return set_err(ctx, L2H_EINVAL, "l2h_matmul: NULL argument");
    if (!type_ok(type)) return set_err(ctx, L2H_ETYPE, "tensor type %d not implemented", type);
    if (ne0 <= 0 || ne1 < 0) return set_err(ctx, L2H_EINVAL, "bad shape");
    if (is_kquant(type) && ne0 % QK_K != 0)
        return set_err(ctx, L2H_EINVAL, "ne0 = %lld is not a multiple of 256", (long long)ne0);
    if (is_kquant(type) && ne0 > L2H_MAX_KQ_INPUT)
        return set_err(ctx, L2H_EINVAL, "a k-quant matrix takes at most %d input features, got %lld", L2H_MAX_KQ_INPUT,
                       (long long)ne0);
    if ((I_sc == nullptr) != (I_min == nullptr)) return set_err(ctx, L2H_EINVAL, "I_sc and I_min go together");
    if (I_sc && !is_kquant(type)) return set_err(ctx, L2H_EINVAL, "integer sums exist for k-quant types only");
    if (ne1 == 0) return L2H_OK;
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevTensor t;
    int rc = dev_tensor_alloc(ctx, type, ne0, ne1, &t);
    if (rc) return rc;
    rc = dev_tensor_upload(ctx, &t, A);
    if (rc == L2H_OK) {
        DevBuf dx, dy, di, dm;
        hipError_t e = dx.alloc((size_t)ne0 * 4);
        if (e == hipSuccess) e = dy.alloc((size_t)ne1 * 4);
        if (e == hipSuccess) e = hipMemcpy(dx.p, x, (size_t)ne0 * 4, hipMemcpyHostToDevice);
        const int64_t nints = ne1 * (ne0 / QK_K);
        if (e == hipSuccess && I_sc) {
            e = di.alloc((size_t)nints * 4);
            if (e == hipSuccess) e = dm.alloc((size_t)nints * 4);
        }
        if (e == hipSuccess) {
            PhaseArgs a{};
            a.max_grid = ctx->prop.multiProcessorCount;
            a.nseg = 1;
            a.w[0] = t;
            a.y[0] = dy.as<float>();
            a.xf = dx.as<float>();
            a.dbg_isc = di.as<int32_t>();
            a.dbg_imin = dm.as<int32_t>();
            e = k_matvec(ctx->stream, a, PRO_QUANT, EPI_STORE);
        }
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e == hipSuccess) e = hipMemcpy(y, dy.p, (size_t)ne1 * 4, hipMemcpyDeviceToHost);
        if (e == hipSuccess && I_sc) {
            e = hipMemcpy(I_sc, di.p, (size_t)nints * 4, hipMemcpyDeviceToHost);
            if (e == hipSuccess) e = hipMemcpy(I_min, dm.p, (size_t)nints * 4, hipMemcpyDeviceToHost);
        }
        if (e != hipSuccess) rc = set_err(ctx, L2H_EHIP, "matmul failed: %s", hipGetErrorString(e));
    }
    dev_tensor_free(&t);
    return rc;
}

// matmul!(y, A, x) with A one of the model's resident matrices (uploaded through l2h_model_set_tensor)
extern "C" int l2h_model_matmul(l2h_model *m, int role, int layer, const float *x, float *y) {
    if (!m || !x || !y) return set_err(m ? m->ctx : nullptr, L2H_EINVAL, "l2h_model_matmul: NULL argument");
    l2h_ctx *ctx = m->ctx;
    if (!m->finalized) return set_err(ctx, L2H_ESTATE, "model not finalized");
    const bool glob = role == L2H_TOK_EMB || role == L2H_OUTPUT;
    const bool per_layer = role >= L2H_WQ && role < L2H_N_ROLES;
    if (!glob && !per_layer) return set_err(ctx, L2H_EINVAL, "role %d is not a matrix", role);
    if (per_layer && (layer < 0 || layer >= m->c.n_layers)) return set_err(ctx, L2H_EINVAL, "layer %d out of range", layer);
    const DevTensor &t = glob ? m->glob[role] : m->L(layer, role);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevBuf dx, dy;
    HIPCHK(ctx, dx.alloc((size_t)t.ne0 * 4));
    HIPCHK(ctx, dy.alloc((size_t)t.ne1 * 4));
    HIPCHK(ctx, hipMemcpy(dx.p, x, (size_t)t.ne0 * 4, hipMemcpyHostToDevice));
    PhaseArgs a{};
    a.max_grid = ctx->prop.multiProcessorCount;
    a.nseg = 1;
    a.w[0] = t;
    a.w[0].layer_stride = 0;  // (the tensor of this very layer: no stepping through the role's slab)
    a.y[0] = dy.as<float>();
    a.xf = dx.as<float>();
    HIPCHK(ctx, k_matvec(ctx->stream, a, PRO_QUANT, EPI_STORE));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipMemcpy(y, dy.p, (size_t)t.ne1 * 4, hipMemcpyDeviceToHost));
    return L2H_OK;
}

extern "C" int l2h_rmsnorm(l2h_ctx *ctx, float *o, const float *x, const float *weight, int64_t n) {
    if (!ctx || !o || !x || !weight) return set_err(ctx, L2H_EINVAL, "l2h_rmsnorm: NULL argument");
    if (n <= 0 || n > 15360) return set_err(ctx, L2H_EINVAL, "length %lld outside 1..15360", (long long)n);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevBuf dx, dw, dout;
    HIPCHK(ctx, dx.alloc((size_t)n * 4));
    HIPCHK(ctx, dw.alloc((size_t)n * 4));
    HIPCHK(ctx, dout.alloc((size_t)n * 4));
    HIPCHK(ctx, hipMemcpy(dx.p, x, (size_t)n * 4, hipMemcpyHostToDevice));
    HIPCHK(ctx, hipMemcpy(dw.p, weight, (size_t)n * 4, hipMemcpyHostToDevice));
    Q8Dev none{nullptr, nullptr, nullptr};
    HIPCHK(ctx, k_stage_dump(ctx->stream, dx.as<float>(), dw.as<float>(), n, PRO_RMSNORM, none, dout.as<float>()));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipMemcpy(o, dout.p, (size_t)n * 4, hipMemcpyDeviceToHost));
    return L2H_OK;
}

// rmsnorm!(o, x, weight) followed by q8_K quantization of o, as the matvec prologue does it
extern "C" int l2h_rmsnorm_q8k(l2h_ctx *ctx, const float *x, const float *weight, int64_t n, void *out_blocks) {
    if (!ctx || !x || !weight || !out_blocks) return set_err(ctx, L2H_EINVAL, "l2h_rmsnorm_q8k: NULL argument");
    if (n <= 0 || n % QK_K != 0 || n > 15360)
        return set_err(ctx, L2H_EINVAL, "length %lld must be a multiple of 256, at most 15360", (long long)n);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevBuf dx, dw;
    HIPCHK(ctx, dx.alloc((size_t)n * 4));
    HIPCHK(ctx, dw.alloc((size_t)n * 4));
    HIPCHK(ctx, hipMemcpy(dx.p, x, (size_t)n * 4, hipMemcpyHostToDevice));
    HIPCHK(ctx, hipMemcpy(dw.p, weight, (size_t)n * 4, hipMemcpyHostToDevice));
    Q8Dev q;
    std::vector<void *> tr;
    int rc = q8_alloc(ctx, n, &q, &tr);
    if (rc) return rc;
    hipError_t e = k_stage_dump(ctx->stream, dx.as<float>(), dw.as<float>(), n, PRO_RMSNORM, q, nullptr);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess)
        rc = q8_pack_blocks(ctx, q, n, out_blocks);
    else
        rc = set_err(ctx, L2H_EHIP, "rmsnorm+quantize failed: %s", hipGetErrorString(e));
    (void)hipFree(tr[0]);
    return rc;
}

extern "C" int l2h_rope(l2h_ctx *ctx, float *x, int head_size, int n_heads, int pos, float freq_base, int neox) {
    if (!ctx || !x) return set_err(ctx, L2H_EINVAL, "l2h_rope: NULL argument");
    if (head_size <= 0 || head_size % 2 != 0 || n_heads <= 0 || pos < 0)
        return set_err(ctx, L2H_EINVAL, "bad rope arguments");
    HIPCHK(ctx, hipSetDevice(ctx->device));
    const size_t bytes = (size_t)head_size * n_heads * 4;
    DevBuf dx;
    HIPCHK(ctx, dx.alloc(bytes));
    HIPCHK(ctx, hipMemcpy(dx.p, x, bytes, hipMemcpyHostToDevice));
    const float theta_scale = powf(freq_base, -(1.0f / (float)(head_size / 2)));
    HIPCHK(ctx, k_rope_only(ctx->stream, dx.as<float>(), head_size, n_heads, pos, theta_scale, neox));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipMemcpy(x, dx.p, bytes, hipMemcpyDeviceToHost));
    return L2H_OK;
}

extern "C" int l2h_softmax(l2h_ctx *ctx, float *x, int64_t n) {
    if (!ctx || !x) return set_err(ctx, L2H_EINVAL, "l2h_softmax: NULL argument");
    if (n <= 0) return set_err(ctx, L2H_EINVAL, "softmax of an empty vector");
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevBuf dx;
    HIPCHK(ctx, dx.alloc((size_t)n * 4));
    HIPCHK(ctx, hipMemcpy(dx.p, x, (size_t)n * 4, hipMemcpyHostToDevice));
    HIPCHK(ctx, k_softmax(ctx->stream, dx.as<float>(), n));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipMemcpy(x, dx.p, (size_t)n * 4, hipMemcpyDeviceToHost));
    return L2H_OK;
}

extern "C" int l2h_attention(l2h_ctx *ctx, float *out, const float *q, const float *kc, const float *vc,
                             int head_size, int n_heads, int n_kv_heads, int pos) {
    if (!ctx || !out || !q || !kc || !vc) return set_err(ctx, L2H_EINVAL, "l2h_attention: NULL argument");
    if (head_size <= 0 || head_size % 4 != 0 || head_size > 1024 || n_heads <= 0 || n_kv_heads <= 0 ||
        n_heads % n_kv_heads != 0 || pos < 0)
        return set_err(ctx, L2H_EINVAL, "bad attention arguments");
    HIPCHK(ctx, hipSetDevice(ctx->device));
    const int np = pos + 1;
    const int seq_len = ((np + L2H_ATT_TILE - 1) / L2H_ATT_TILE) * L2H_ATT_TILE;
    const int dim = head_size * n_heads, kv_dim = head_size * n_kv_heads;
    const int ntiles = seq_len / L2H_ATT_TILE;
    DevBuf dq, dqd, dkl, dvl, dkc, dvc, datt, dpd, dpart, dout, dctl;
    HIPCHK(ctx, dq.alloc((size_t)dim * 4));
    HIPCHK(ctx, dqd.alloc((size_t)dim * 8));
    HIPCHK(ctx, dkl.alloc((size_t)np * kv_dim * 4));
    HIPCHK(ctx, dvl.alloc((size_t)np * kv_dim * 4));
    HIPCHK(ctx, dkc.alloc((size_t)seq_len * kv_dim * 4));
    HIPCHK(ctx, dvc.alloc((size_t)seq_len * kv_dim * 4));
    HIPCHK(ctx, datt.alloc((size_t)seq_len * n_heads * 4));
    HIPCHK(ctx, dpd.alloc((size_t)seq_len * n_heads * 8));
    HIPCHK(ctx, dpart.alloc((size_t)ntiles * dim * 8));
    HIPCHK(ctx, dout.alloc((size_t)dim * 4));
    HIPCHK(ctx, dctl.alloc(sizeof(DecodeCtl)));
    DecodeCtl h{};
    h.pos = pos;
    HIPCHK(ctx, hipMemcpy(dctl.p, &h, sizeof h, hipMemcpyHostToDevice));
    HIPCHK(ctx, hipMemcpy(dq.p, q, (size_t)dim * 4, hipMemcpyHostToDevice));
    HIPCHK(ctx, hipMemcpy(dkl.p, kc, (size_t)np * kv_dim * 4, hipMemcpyHostToDevice));
    HIPCHK(ctx, hipMemcpy(dvl.p, vc, (size_t)np * kv_dim * 4, hipMemcpyHostToDevice));
    HIPCHK(ctx, k_f32_to_f64(ctx->stream, dq.as<float>(), dqd.as<double>(), dim));
    HIPCHK(ctx, k_kv_layout(ctx->stream, dkc.as<float>(), dvc.as<float>(), dkl.as<float>(), dvl.as<float>(), 0, np,
                            head_size, n_kv_heads, seq_len, true, 0));
    HIPCHK(ctx, k_attention(ctx->stream, dqd.as<double>(), dkc.as<float>(), dvc.as<float>(), datt.as<float>(),
                            dpd.as<double>(), dpart.as<double>(), dout.as<float>(), (const DecodeCtl *)dctl.p,
                            head_size, n_heads, n_kv_heads, seq_len, 0));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipMemcpy(out, dout.p, (size_t)dim * 4, hipMemcpyDeviceToHost));
    return L2H_OK;
}

extern "C" int l2h_swiglu(l2h_ctx *ctx, float *hb, const float *hb2, int64_t n) {
    if (!ctx || !hb || !hb2) return set_err(ctx, L2H_EINVAL, "l2h_swiglu: NULL argument");
    if (n <= 0 || n > (1 << 30)) return set_err(ctx, L2H_EINVAL, "bad length");
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevBuf a, b;
    HIPCHK(ctx, a.alloc((size_t)n * 4));
    HIPCHK(ctx, b.alloc((size_t)n * 4));
    HIPCHK(ctx, hipMemcpy(a.p, hb, (size_t)n * 4, hipMemcpyHostToDevice));
    HIPCHK(ctx, hipMemcpy(b.p, hb2, (size_t)n * 4, hipMemcpyHostToDevice));
    HIPCHK(ctx, k_swiglu(ctx->stream, a.as<float>(), b.as<float>(), (int)n));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipMemcpy(hb, a.p, (size_t)n * 4, hipMemcpyDeviceToHost));
    return L2H_OK;
}

extern "C" int l2h_argmax(l2h_ctx *ctx, const float *x, int64_t n, int32_t *out) {
    if (!ctx || !x || !out) return set_err(ctx, L2H_EINVAL, "l2h_argmax: NULL argument");
    if (n <= 0 || n > 0x7FFFFFFF) return set_err(ctx, L2H_EINVAL, "bad length");
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevBuf dx, dp, dctl, dout;
    HIPCHK(ctx, dx.alloc((size_t)n * 4));
    HIPCHK(ctx, dp.alloc((size_t)L2H_ARGMAX_BLOCKS * 8));
    HIPCHK(ctx, dctl.alloc(sizeof(DecodeCtl)));
    HIPCHK(ctx, dout.alloc(4));
    DecodeCtl h{};
    h.n_prompt = 1;
    HIPCHK(ctx, hipMemcpy(dctl.p, &h, sizeof h, hipMemcpyHostToDevice));
    HIPCHK(ctx, hipMemcpy(dx.p, x, (size_t)n * 4, hipMemcpyHostToDevice));
    HIPCHK(ctx, k_argmax(ctx->stream, dx.as<float>(), n, dp.as<int64_t>(), (DecodeCtl *)dctl.p, dout.as<int32_t>(), 1));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipMemcpy(out, dout.p, 4, hipMemcpyDeviceToHost));
    return L2H_OK;
}

// l2h_argmax on device memory, without a single allocation: the keys of the first stage live in a static device
// array whose address on this context's device was looked up at l2h_ctx_create.
extern "C" int l2h_argmax_noalloc(l2h_ctx *ctx, const float *x_dev, int64_t n, int32_t *out_dev) {
    if (!ctx || !x_dev || !out_dev) return set_err(ctx, L2H_EINVAL, "l2h_argmax_noalloc: NULL argument");
    if (n <= 0 || n > L2H_ARGMAX_NOALLOC_MAX_N)
        return set_err(ctx, L2H_EINVAL, "l2h_argmax_noalloc: n = %lld outside 1..%lld", (long long)n,
                       (long long)L2H_ARGMAX_NOALLOC_MAX_N);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    HIPCHK(ctx, k_argmax_noalloc(ctx->stream, ctx->device, x_dev, n, out_dev));
    return L2H_OK;
}

// ------------------------------------------------------------------------------------------
// measurement
// ------------------------------------------------------------------------------------------
extern "C" int l2h_profile_matvec(l2h_model *m, int role, int iters, float *avg_us, int64_t *bytes) {
    if (!m || !avg_us) return L2H_EINVAL;
    l2h_ctx *ctx = m->ctx;
    if (!m->finalized) return set_err(ctx, L2H_ESTATE, "model not finalized");
    if (iters < 1) return set_err(ctx, L2H_EINVAL, "iters must be >= 1");
    if (role != L2H_WQ && role != L2H_WO && role != L2H_W1 && role != L2H_W2 && role != L2H_OUTPUT)
        return set_err(ctx, L2H_EINVAL, "role %d has no matvec launch of its own", role);
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DecodeCtl h{};  // position 0: the q/k/v launch appends to cache row 0
    HIPCHK(ctx, hipMemcpy(m->ctl, &h, sizeof h, hipMemcpyHostToDevice));
    const int n_layers = role == L2H_OUTPUT ? 1 : m->c.n_layers;
    int64_t b = 0;
    if (role == L2H_WQ)
        b = m->L(0, L2H_WQ).gguf_bytes + m->L(0, L2H_WK).gguf_bytes + m->L(0, L2H_WV).gguf_bytes;
    else if (role == L2H_W1)
        b = m->L(0, L2H_W1).gguf_bytes + m->L(0, L2H_W3).gguf_bytes;
    else if (role == L2H_OUTPUT)
        b = m->glob[L2H_OUTPUT].gguf_bytes;
    else
        b = m->L(0, role).gguf_bytes;
    hipEvent_t e0, e1;
    HIPCHK(ctx, hipEventCreate(&e0));
    HIPCHK(ctx, hipEventCreate(&e1));
    for (int pass = 0; pass < 2; pass++) {  // pass 0 warms up
        const int reps = pass == 0 ? 1 : iters;
        if (pass == 1) HIPCHK(ctx, hipEventRecord(e0, ctx->stream));
        for (int it = 0; it < reps; it++) {
            for (int l = 0; l < n_layers; l++) {
                hipError_t e;
                switch (role) {
                case L2H_WQ: e = launch_qkv(m, l); break;
                case L2H_WO: e = launch_wo(m, l); break;
                case L2H_W1: e = launch_w13(m, l); break;
                case L2H_W2: e = launch_w2(m, l); break;
                default: e = launch_output(m); break;
                }
                if (e != hipSuccess) return set_err(ctx, L2H_EHIP, "matvec launch failed: %s", hipGetErrorString(e));
            }
        }
        if (pass == 1) HIPCHK(ctx, hipEventRecord(e1, ctx->stream));
        HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    }
    float ms = 0.0f;
    HIPCHK(ctx, hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *avg_us = ms * 1000.0f / (float)(iters * n_layers);
    if (bytes) *bytes = b;
    return L2H_OK;
}

extern "C" int l2h_profile_stream_read(l2h_ctx *ctx, int64_t n_bytes, int iters, float *avg_us) {
    if (!ctx || !avg_us) return L2H_EINVAL;
    if (n_bytes < 16 || iters < 1) return set_err(ctx, L2H_EINVAL, "bad arguments");
    HIPCHK(ctx, hipSetDevice(ctx->device));
    DevBuf buf, sink;
    HIPCHK(ctx, buf.alloc((size_t)n_bytes));
    HIPCHK(ctx, sink.alloc(16));
    HIPCHK(ctx, hipMemset(buf.p, 1, (size_t)n_bytes));
    hipEvent_t e0, e1;
    HIPCHK(ctx, hipEventCreate(&e0));
    HIPCHK(ctx, hipEventCreate(&e1));
    HIPCHK(ctx, k_stream_read(ctx->stream, buf.as<uint4>(), n_bytes / 16, sink.as<uint32_t>()));
    HIPCHK(ctx, hipEventRecord(e0, ctx->stream));
    for (int i = 0; i < iters; i++)
        HIPCHK(ctx, k_stream_read(ctx->stream, buf.as<uint4>(), n_bytes / 16, sink.as<uint32_t>()));
    HIPCHK(ctx, hipEventRecord(e1, ctx->stream));
    HIPCHK(ctx, hipEventSynchronize(e1));
    float ms = 0.0f;
    HIPCHK(ctx, hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *avg_us = ms * 1000.0f / (float)iters;
    return L2H_OK;
}

#ifdef L2H_TIMELINE
// profiling build only: wall-clock stamps (100 MHz) of the last persistent-kernel launch
extern "C" int l2h_debug_timeline(l2h_model *m, long long *out, int n_wg) {
    if (!m || !(m->mega || m->flow) || !m->timeline) return L2H_ESTATE;
    HIPCHK(m->ctx, hipMemcpy(out, m->timeline, ((size_t)n_wg * 64 + (m->flow ? 1024 : 0)) * 8, hipMemcpyDeviceToHost));
    return L2H_OK;
}
extern "C" int l2h_debug_timeline2(l2h_model *m, long long *out, int n_wg) {
    if (!m || !m->mega || !m->timeline2) return L2H_ESTATE;
    HIPCHK(m->ctx, hipMemcpy(out, m->timeline2, (size_t)n_wg * 8 * 8, hipMemcpyDeviceToHost));
    return L2H_OK;
}
#endif

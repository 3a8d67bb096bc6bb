// Small per-token kernels: weight repack, embedding lookup, rmsnorm + q8_K quantize,
// SwiGLU + quantize, RoPE + KV append, argmax, layout helpers.
#include <hip/hip_fp16.h>
#include <mutex>

#include "dev_common.h"

// ------------------------------------------------------------------------------------------
// Repack GGUF super-blocks <-> field streams (see DevTensor).  One thread per 16-bit word
// of the raw block keeps it valid for q6_K, whose 210-byte blocks are only 2-byte aligned.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ int64_t stream_word_index(int type, int64_t blk, int w, int &which) {
    // returns the index (in 16-bit words) inside stream `which` for word w of block blk
    // which: 0 hdr, 1 qs/ql, 2 qh, 3 sc6, 4 d6
    if (type == L2H_TYPE_Q4_K) {
        if (w < 8) { which = 0; return blk * 8 + w; }
        which = 1; return blk * 64 + (w - 8);
    }
    if (type == L2H_TYPE_Q5_K) {
        if (w < 8) { which = 0; return blk * 8 + w; }
        if (w < 24) { which = 2; return blk * 16 + (w - 8); }
        which = 1; return blk * 64 + (w - 24);
    }
    // Q6_K: ql 64 words, qh 32 words, scales 8 words (bytes permuted, handled by caller), d 1 word
    if (w < 64) { which = 1; return blk * 64 + w; }
    if (w < 96) { which = 2; return blk * 32 + (w - 64); }
    if (w < 104) { which = 3; return blk * 8 + (w - 96); }
    which = 4; return blk;
}

__global__ __launch_bounds__(256) void repack_kernel(DevTensor t, const uint16_t *raw, uint16_t *raw_out,
                                                     int64_t nblocks, int words_per_block, bool inverse) {
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= nblocks * words_per_block) return;
    const int64_t blk = gid / words_per_block;
    const int w = (int)(gid % words_per_block);
    int which;
    const int64_t idx = stream_word_index(t.type, blk, w, which);
    uint16_t *streams[5] = {(uint16_t *)t.hdr, (uint16_t *)t.qs, (uint16_t *)t.qh, (uint16_t *)t.sc6,
                            (uint16_t *)t.d6};
    if (which == 3) {
        // q6_K scales: original byte o = 8n + hh + 2g  <->  stream byte p = 4*(2n+hh) + g
        uint8_t *sc = (uint8_t *)t.sc6 + blk * 16;
        const uint8_t *rb = (const uint8_t *)raw + blk * 210 + 192;
        uint8_t *ro = (uint8_t *)raw_out + blk * 210 + 192;
        for (int k = 0; k < 2; k++) {
            const int o = 2 * (w - 96) + k;
            const int n = o >> 3, hh = o & 1, g = (o & 7) >> 1;
            const int p = 4 * (2 * n + hh) + g;
            if (inverse)
                ro[o] = sc[p];
            else
                sc[p] = rb[o];
        }
        return;
    }
    if (inverse)
        raw_out[gid] = streams[which][idx];
    else
        streams[which][idx] = raw[gid];
}

hipError_t k_repack(hipStream_t s, const DevTensor &t, const void *raw_dev, bool inverse, void *raw_out) {
    const int wpb = (int)(l2h_gguf_block_bytes(t.type) / 2);
    const int64_t nblocks = t.ne1 * t.nb;
    const int64_t total = nblocks * wpb;
    const int64_t grid = (total + 255) / 256;
    hipLaunchKernelGGL(repack_kernel, dim3((unsigned)grid), dim3(256), 0, s, t, (const uint16_t *)raw_dev,
                       (uint16_t *)raw_out, nblocks, wpb, inverse);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// dequantize!(x, token_embedding_table[:, token])  (reference src/inference.jl:236)
// The token of the step is prompt[step] while inside the prompt, else the previous argmax
// (src/inference.jl:354-360,385).
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void embed_kernel(DevTensor emb, const DecodeCtl *ctl, const int32_t *prompt,
                                                    float *x, float *rope_cs, int hs, float theta_scale) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (blockIdx.x == 0 && threadIdx.x < (hs >> 1)) {
        // cos/sin of this position's RoPE angles, shared by all layers and heads: theta_i is
        // fp32(pos) advanced by i fp32 multiplications (reference src/inference.jl:122-127)
        float theta = 1.0f * (float)ctl->pos;
        for (int k = 0; k < (int)threadIdx.x; k++) theta *= theta_scale;
        rope_cs[2 * threadIdx.x] = (float)cos((double)theta);
        rope_cs[2 * threadIdx.x + 1] = (float)sin((double)theta);
    }
    if (i >= emb.ne0) return;
    const int tok = ctl->step < ctl->n_prompt ? prompt[ctl->step] : ctl->last_argmax;
    x[i] = dequant_elem(emb, tok, i);
}

hipError_t k_embed(hipStream_t s, const DevTensor &emb, const DecodeCtl *ctl, const int32_t *prompt, float *x,
                   float *rope_cs, int head_size, float theta_scale) {
    hipLaunchKernelGGL(embed_kernel, dim3((unsigned)((emb.ne0 + 255) / 256)), dim3(256), 0, s, emb, ctl, prompt, x,
                       rope_cs, head_size, theta_scale);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void dequant_kernel(DevTensor t, int64_t row0, int64_t nrows, float *y) {
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= nrows * t.ne0) return;
    y[gid] = dequant_elem(t, row0 + gid / t.ne0, gid % t.ne0);
}

hipError_t k_dequant(hipStream_t s, const DevTensor &t, int64_t row0, int64_t nrows, float *y) {
    const int64_t total = nrows * t.ne0;
    hipLaunchKernelGGL(dequant_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, t, row0, nrows, y);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// hb[i] = hb[i] * (1/(1+exp(-hb[i]))) * hb2[i]  (reference src/inference.jl:295-299),
// exp evaluated in fp64 and rounded to fp32.  Stand-alone form, used when w1 and w3 differ in
// type and cannot share one launch.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void swiglu_kernel(float *hb, const float *hb2, int n) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n) return;
    const float a = hb[t];
    const float e = (float)exp((double)(-a));
    const float v = a * (1.0f / (1.0f + e));
    hb[t] = v * hb2[t];
}

hipError_t k_swiglu(hipStream_t s, float *hb, const float *hb2, int n) {
    hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, hb, hb2, n);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// rope!(x) (reference src/inference.jl:112-167), stand-alone form.
// theta of pair i is fp32(pos) advanced by i fp32 multiplications with theta_scale
// (:122-127); cos/sin are evaluated in fp64 and rounded to fp32; the complex product
// rounds each of its four products (Complex{Float32} multiplication).
// K cache layout per layer: [n_kv_heads][hs/4][seq_len][4]; V cache: [n_kv_heads][seq_len][hs].
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ void rope_pair(float a, float b, int i, int pos, float theta_scale, float &re, float &im) {
    float theta = 1.0f * (float)pos;
    for (int k = 0; k < i; k++) theta *= theta_scale;
    const float c = (float)cos((double)theta);
    const float s = (float)sin((double)theta);
    const float ac = a * c, bs = b * s, as = a * s, bc = b * c;
    re = ac - bs;
    im = as + bc;
}

__device__ __forceinline__ int64_t kc_index(int kvh, int i, int t, int hs, int seq_len) {
    return (((int64_t)kvh * (hs >> 2) + (i >> 2)) * seq_len + t) * 4 + (i & 3);
}

__global__ __launch_bounds__(256) void rope_only_kernel(float *x, int hs, int n_heads, int pos, float theta_scale,
                                                        int neox) {
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int half = hs >> 1;
    if (gid >= n_heads * half) return;
    const int h = gid / half, i = gid % half;
    const int e0 = neox ? i : 2 * i, e1 = neox ? half + i : 2 * i + 1;
    float re, im;
    rope_pair(x[h * hs + e0], x[h * hs + e1], i, pos, theta_scale, re, im);
    x[h * hs + e0] = re;
    x[h * hs + e1] = im;
}

hipError_t k_rope_only(hipStream_t s, float *x, int head_size, int n_heads, int pos, float theta_scale, int neox) {
    const int total = n_heads * head_size / 2;
    hipLaunchKernelGGL(rope_only_kernel, dim3((total + 255) / 256), dim3(256), 0, s, x, head_size, n_heads, pos,
                       theta_scale, neox);
    return hipGetLastError();
}

// canonical [n][kv_dim] rows <-> cache layouts, positions pos0 .. pos0+n-1 of one layer
__global__ __launch_bounds__(256) void kv_layout_kernel(float *kc, float *vc, float *k_lin, float *v_lin, int pos0,
                                                        int n, int hs, int n_kv_heads, int seq_len, int to_cache, int kv16) {
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int kv_dim = hs * n_kv_heads;
    if (gid >= (int64_t)n * kv_dim) return;
    const int r = (int)(gid / kv_dim), e = (int)(gid % kv_dim);
    const int h = e / hs, i = e % hs, t = pos0 + r;
    const int64_t ki = kc_index(h, i, t, hs, seq_len);
    const int64_t vi = ((int64_t)h * seq_len + t) * hs + i;
    if (kv16) {  // fp16 cache: rounded to nearest even on the way in, widened exactly on the way out
        __half *kh = (__half *)kc, *vh = (__half *)vc;
        const int64_t ki = kc16_index(h, i, t, hs, seq_len);  // (the fp16 K cache groups eight elements)
        if (to_cache) {
            kh[ki] = __float2half_rn(k_lin[gid]);
            vh[vi] = __float2half_rn(v_lin[gid]);
        } else {
            k_lin[gid] = __half2float(kh[ki]);
            v_lin[gid] = __half2float(vh[vi]);
        }
        return;
    }
    if (to_cache) {
        kc[ki] = k_lin[gid];
        vc[vi] = v_lin[gid];
    } else {
        k_lin[gid] = kc[ki];
        v_lin[gid] = vc[vi];
    }
}

hipError_t k_kv_layout(hipStream_t s, float *kc, float *vc, float *k_lin, float *v_lin, int pos0, int n, int head_size,
                       int n_kv_heads, int seq_len, bool to_cache, int kv16) {
    const int64_t total = (int64_t)n * head_size * n_kv_heads;
    hipLaunchKernelGGL(kv_layout_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, kc, vc, k_lin, v_lin,
                       pos0, n, head_size, n_kv_heads, seq_len, to_cache ? 1 : 0, kv16);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// argmax(logits): first maximal index (reference src/inference.jl:360).  Keys order by
// value, then by lower index; stage 2 also advances the control block to the next step.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned long long argmax_key(float v, uint32_t idx) {
    uint32_t b = __float_as_uint(v);
    b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    if (v == 0.0f) b = 0x80000000u;  // -0.0 and +0.0 compare equal
    return ((unsigned long long)b << 32) | (unsigned long long)(0xFFFFFFFFu - idx);
}

__device__ __forceinline__ unsigned long long block_max_u64(unsigned long long key, unsigned long long *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const unsigned long long o = __shfl_xor(key, m, WAVE);
        key = o > key ? o : key;
    }
    __syncthreads();
    if (lane == 0) red[wave] = key;
    __syncthreads();
    unsigned long long t = red[0];
    for (int w = 1; w < nw; w++) t = red[w] > t ? red[w] : t;
    return t;
}

__global__ __launch_bounds__(256) void argmax_stage1_kernel(const float *x, int64_t n, unsigned long long *partial) {
    __shared__ unsigned long long red[4];
    unsigned long long best = 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const unsigned long long key = argmax_key(x[i], (uint32_t)i);
        best = key > best ? key : best;
    }
    best = block_max_u64(best, red);
    if (threadIdx.x == 0) partial[blockIdx.x] = best;
}

__global__ __launch_bounds__(256) void argmax_stage2_kernel(const unsigned long long *partial, int nparts,
                                                            DecodeCtl *ctl, int32_t *out_tokens, int max_out) {
    __shared__ unsigned long long red[4];
    unsigned long long best = 0;
    for (int i = threadIdx.x; i < nparts; i += blockDim.x) best = partial[i] > best ? partial[i] : best;
    best = block_max_u64(best, red);
    if (threadIdx.x == 0) {
        const int idx = (int)(0xFFFFFFFFu - (uint32_t)(best & 0xFFFFFFFFull));
        ctl->last_argmax = idx;
        if (ctl->step >= ctl->n_prompt - 1 && ctl->n_out < max_out) {
            out_tokens[ctl->n_out] = idx;
            ctl->n_out += 1;
        }
        ctl->step += 1;
        ctl->pos += 1;
    }
}

hipError_t k_argmax(hipStream_t s, const float *x, int64_t n, int64_t *partial, DecodeCtl *ctl, int32_t *out_tokens,
                    int max_out) {
    hipLaunchKernelGGL(argmax_stage1_kernel, dim3(L2H_ARGMAX_BLOCKS), dim3(256), 0, s, x, n,
                       (unsigned long long *)partial);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(argmax_stage2_kernel, dim3(1), dim3(256), 0, s, (const unsigned long long *)partial,
                       L2H_ARGMAX_BLOCKS, ctl, out_tokens, max_out);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// argmax for callers that cannot allocate (code under stream capture, serving loops, harnesses that forbid
// hipMalloc): the same two stages, with the per-workgroup keys of stage 1 in a file-scope device array
// instead of an allocation.  Every GPU the library runs on holds its own copy of the array (2 KiB) until
// the process ends; calls that overlap on one GPU would share it and race.
// ------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned long long scratch[L2H_ARGMAX_BLOCKS];

// In host code `scratch` is a stand-in, not a device address: each device's address is asked for once, with
// that device current, and kept.
#define L2H_MAX_DEVICES 64
static unsigned long long *g_scratch_ptr[L2H_MAX_DEVICES];

static std::mutex g_scratch_mu;

hipError_t k_noalloc_init(int device) {
    if (device < 0 || device >= L2H_MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[device]) return hipSuccess;
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[device] = (unsigned long long *)p;
    return hipSuccess;
}

__global__ __launch_bounds__(256) void argmax_stage2_plain_kernel(const unsigned long long *partial, int nparts,
                                                                  int32_t *out) {
    __shared__ unsigned long long red[4];
    unsigned long long best = 0;
    for (int i = threadIdx.x; i < nparts; i += blockDim.x) best = partial[i] > best ? partial[i] : best;
    best = block_max_u64(best, red);
    if (threadIdx.x == 0) *out = (int32_t)(0xFFFFFFFFu - (uint32_t)(best & 0xFFFFFFFFull));
}

// x and out are device pointers; nothing is allocated, nothing is waited for.  Stage 1 writes every one of
// the L2H_ARGMAX_BLOCKS keys on every call (a workgroup without elements writes the smallest key), so what
// the previous call left in the array is never read.
hipError_t k_argmax_noalloc(hipStream_t s, int device, const float *x, int64_t n, int32_t *out) {
    if (device < 0 || device >= L2H_MAX_DEVICES || !g_scratch_ptr[device]) return hipErrorNotInitialized;
    unsigned long long *partial = g_scratch_ptr[device];
    hipLaunchKernelGGL(argmax_stage1_kernel, dim3(L2H_ARGMAX_BLOCKS), dim3(256), 0, s, x, n, partial);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(argmax_stage2_plain_kernel, dim3(1), dim3(256), 0, s, (const unsigned long long *)partial,
                       L2H_ARGMAX_BLOCKS, out);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// softmax!(x) (reference src/inference.jl:169-174), single vector, one workgroup.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void softmax_kernel(float *x, int64_t n) {
    __shared__ double redd[16];
    __shared__ float redf[16];
    float mx = -INFINITY;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) mx = fmaxf(mx, x[i]);
    mx = block_max_f32(mx, redf);
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float e = (float)exp((double)(x[i] - mx));
        x[i] = e;
        acc += (double)e;
    }
    const float sf = (float)block_sum_f64(acc, redd);
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) x[i] = x[i] / sf;
}

hipError_t k_softmax(hipStream_t s, float *x, int64_t n) {
    hipLaunchKernelGGL(softmax_kernel, dim3(1), dim3(256), 0, s, x, n);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// plain streaming read (measured HBM ceiling) and fp32 -> fp64 widening
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4 *p, int64_t n16, uint32_t *sink) {
    uint32_t acc = 0;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const uint4 a = p[i], b = p[i + stride], c = p[i + 2 * stride], d = p[i + 3 * stride];
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    for (; i < n16; i += stride) {
        const uint4 a = p[i];
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;  // practically never true: keeps the loads alive
}

hipError_t k_stream_read(hipStream_t s, const uint4 *p, int64_t n16, uint32_t *sink) {
    hipLaunchKernelGGL(stream_read_kernel, dim3(256 * 8), dim3(256), 0, s, p, n16, sink);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void f32_to_f64_kernel(const float *x, double *y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = (double)x[i];
}

hipError_t k_f32_to_f64(hipStream_t s, const float *x, double *y, int64_t n) {
    hipLaunchKernelGGL(f32_to_f64_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, y, n);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// temperature sampling (reference src/inference.jl:363-367): logits ./= T; softmax!; wsample.
// wsample's walk is reproduced with a host-supplied uniform number u in [0, 1): the pick is the first
// index whose cumulative weight reaches u * sum(weights).  exp in fp64 rounded to fp32 and the sums
// in fp64 (as everywhere in this library); one workgroup, thread t owns a contiguous slice.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void sample_kernel(const float *logits, int n, float temperature, float u,
                                                      float *p, int32_t *out) {
    __shared__ double redd[16];
    __shared__ float redf[16];
    __shared__ double s_cum[1025];
    const int tid = threadIdx.x;
    const int per = (n + 1023) / 1024, lo = min(n, tid * per), hi = min(n, lo + per);
    float mx = -INFINITY;
    for (int i = lo; i < hi; i++) {
        const float v = logits[i] / temperature;
        p[i] = v;
        mx = fmaxf(mx, v);
    }
    mx = block_max_f32(mx, redf);
    double sum = 0.0;
    for (int i = lo; i < hi; i++) {
        const float e = (float)exp((double)(p[i] - mx));
        p[i] = e;
        sum += (double)e;
    }
    const float sf = (float)block_sum_f64(sum, redd);
    double mine = 0.0;
    for (int i = lo; i < hi; i++) {
        const float pr = p[i] / sf;
        p[i] = pr;
        mine += (double)pr;
    }
    s_cum[tid + 1] = mine;
    __syncthreads();
    if (tid == 0) {
        s_cum[0] = 0.0;
        for (int k = 1; k <= 1024; k++) s_cum[k] += s_cum[k - 1];
    }
    __syncthreads();
    const double target = (double)u * s_cum[1024];
    // the slice in which the cumulative weight first reaches the target (the last non-empty one if
    // rounding leaves the target just above the total)
    const bool here = lo < hi && s_cum[tid] < target && (target <= s_cum[tid + 1] || hi == n);
    const bool first_zero = tid == 0 && target <= 0.0;
    if (here || first_zero) {
        double cw = s_cum[tid];
        int pick = hi - 1;
        for (int i = lo; i < hi; i++) {
            cw += (double)p[i];
            if (cw >= target) {
                pick = i;
                break;
            }
        }
        *out = pick;
    }
}

hipError_t k_sample(hipStream_t s, const float *logits, int n, float temperature, float u, float *p, int32_t *out) {
    hipLaunchKernelGGL(sample_kernel, dim3(1), dim3(1024), 0, s, logits, n, temperature, u, p, out);
    return hipGetLastError();
}

// Decode attention for one position (reference src/inference.jl:176-220, 263-278):
//   scores   att[h][t] = fp32(sum_fp64 q[h][i]*K[t][i]) / sqrt(hs)      attention_weights!, :268
//   softmax  per head: max, exp (fp64, rounded to fp32), fp64 sum, p = e / sum   softmax!
//   values   out[h][i] = fp32(sum_fp64 p[h][t]*V[t][i])                 combine_values!
// Grids are sized for seq_len and exit early past the current position, so one recorded
// launch sequence serves every position.
// K cache layout per layer: [n_kv_heads][hs/4][seq_len][4] (a lane per timestep reads
// contiguous 16-byte pieces); V cache: [n_kv_heads][seq_len][hs] (a lane per feature).
#include "matvec_dev.h"

#ifndef L2H_AV_MIN_WGS
#define L2H_AV_MIN_WGS 1024  // the value pass splits a full cache over at least this many workgroups (512: 0.5 % slower, 2048: 2 %)
#endif

// One wavefront: 64 consecutive timesteps of GH query heads that share one KV head.
template <int GH>
__global__ __launch_bounds__(256) void attn_scores_kernel(const double *qd, const float *kc, float *att,
                                                          const DecodeCtl *ctl, int hs, int n_heads, int n_kv_heads,
                                                          int seq_len) {
    const int pos = ctl->pos;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tile = blockIdx.x * 4 + wave;
    const int t = tile * L2H_ATT_TILE + lane;
    if (tile * L2H_ATT_TILE > pos) return;
    const int h0 = blockIdx.y * GH;
    const int kvh = h0 / (n_heads / n_kv_heads);
    if (t > pos) return;
    const float4 *kp = (const float4 *)kc + (int64_t)kvh * (hs >> 2) * seq_len + t;
    double acc[GH];
#pragma unroll
    for (int g = 0; g < GH; g++) acc[g] = 0.0;
    for (int i4 = 0; i4 < (hs >> 2); i4++) {
        const float4 kv = kp[(int64_t)i4 * seq_len];
        const double k0 = (double)kv.x, k1 = (double)kv.y, k2 = (double)kv.z, k3 = (double)kv.w;
#pragma unroll
        for (int g = 0; g < GH; g++) {
            const double *qq = qd + (int64_t)(h0 + g) * hs + 4 * i4;
            acc[g] = fma(qq[0], k0, acc[g]);
            acc[g] = fma(qq[1], k1, acc[g]);
            acc[g] = fma(qq[2], k2, acc[g]);
            acc[g] = fma(qq[3], k3, acc[g]);
        }
    }
    const float scale = sqrtf((float)hs);
#pragma unroll
    for (int g = 0; g < GH; g++) att[(int64_t)(h0 + g) * seq_len + t] = (float)acc[g] / scale;
}

// One workgroup per head: softmax over att[h][0..pos]; probabilities written as fp32 (att)
// and widened to fp64 (pd) for the value pass.
__global__ __launch_bounds__(1024) void attn_softmax_kernel(float *att, double *pd, const DecodeCtl *ctl, int seq_len) {
    __shared__ double redd[16];
    __shared__ float redf[16];
    const int n = ctl->pos + 1;
    float *x = att + (int64_t)blockIdx.x * seq_len;
    double *p = pd + (int64_t)blockIdx.x * seq_len;
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < n; i += blockDim.x) mx = fmaxf(mx, x[i]);
    mx = block_max_f32(mx, redf);
    double acc = 0.0;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float e = (float)exp((double)(x[i] - mx));
        x[i] = e;
        acc += (double)e;
    }
    const float sf = (float)block_sum_f64(acc, redd);
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float pr = x[i] / sf;
        x[i] = pr;
        p[i] = (double)pr;
    }
}

// One workgroup (hs threads): 64 timesteps of GH heads sharing a KV head -> fp64 partial sums.
template <int GH>
__global__ void attn_av_kernel(const double *pd, const float *vc, double *part, const DecodeCtl *ctl, int hs,
                               int n_heads, int n_kv_heads, int seq_len) {
    const int pos = ctl->pos;
    const int split = blockIdx.x;
    const int t0 = split * L2H_ATT_TILE;
    if (t0 > pos) return;
    const int t1 = min(t0 + L2H_ATT_TILE, pos + 1);
    const int h0 = blockIdx.y * GH;
    const int kvh = h0 / (n_heads / n_kv_heads);
    const int i = threadIdx.x;
    const float *vp = vc + (int64_t)kvh * seq_len * hs + i;
    double acc[GH];
#pragma unroll
    for (int g = 0; g < GH; g++) acc[g] = 0.0;
    for (int t = t0; t < t1; t++) {
        const double v = (double)vp[(int64_t)t * hs];
#pragma unroll
        for (int g = 0; g < GH; g++) acc[g] = fma(pd[(int64_t)(h0 + g) * seq_len + t], v, acc[g]);
    }
#pragma unroll
    for (int g = 0; g < GH; g++) part[((int64_t)split * n_heads + h0 + g) * hs + i] = acc[g];
}

// out[e] = fp32(sum over splits of the partial sums)
__global__ __launch_bounds__(256) void attn_reduce_kernel(const double *part, float *out, const DecodeCtl *ctl,
                                                          int dim) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= dim) return;
    const int nsplit = ctl->pos / L2H_ATT_TILE + 1;
    double acc = 0.0;
    for (int s = 0; s < nsplit; s++) acc += part[(int64_t)s * dim + e];
    out[e] = (float)acc;
}

// ---- long caches: launches sized to fill the chip (scores, exponentials, values, final sum) ----
// Scores: a workgroup = 64 timesteps of GH heads that share a KV head; wavefront w takes quarter w
// of the head dimension (all of its 16-byte loads in flight at once), the quarters are added in
// fixed order through LDS.
template <int GH, bool H16>
__global__ __launch_bounds__(256) void attn_scores4_kernel(const double *qd, const float *kc, float *att, float *tmax,
                                                           const DecodeCtl *ctl, int hs, int n_heads, int n_kv_heads,
                                                           int seq_len) {
    __shared__ double s_q[GH * 128];
    __shared__ double s_part[4][GH][64];
    const int pos = ctl->pos;
    const int t0 = blockIdx.x * 64;
    if (t0 > pos) return;
    const int lane = threadIdx.x & 63, part = threadIdx.x >> 6;
    const int h0 = blockIdx.y * GH, kvh = h0 / (n_heads / n_kv_heads);
    for (int i = threadIdx.x; i < GH * hs; i += 256) s_q[(i / hs) * 128 + i % hs] = qd[(int64_t)h0 * hs + i];
    const int t = min(t0 + lane, pos);
    double acc[GH];
#pragma unroll
    for (int g = 0; g < GH; g++) acc[g] = 0.0;
    if constexpr (H16) {
        // fp16 cache: 16-byte groups of eight elements, hs / 32 of them per quarter (hs a multiple of 32, at most 128)
        const int per8 = hs >> 5;
        const int64_t kg = ((int64_t)kvh * (hs >> 3) + part * per8) * seq_len + t;
        // (all loads are requested before one is waited for: no branch around a load — a group beyond the head size
        // repeats group 0 — and the widening to fp32 comes after the last request)
        h8_bits kb[4];
#pragma unroll
        for (int u = 0; u < 4; u++) kb[u] = ldg_nt_h8_bits(kc, kg + (int64_t)(u < per8 ? u : 0) * seq_len);
        Half8 kv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) kv[u] = h8_widen(kb[u]);
        __syncthreads();
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (u < per8) {
#pragma unroll
                for (int g = 0; g < GH; g++) {
                    const double *qq = s_q + g * 128 + 8 * (part * per8 + u);
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[g] = fma(qq[e], (double)kv[u].v[e], acc[g]);
                }
            }
        }
    } else {
        const int per = hs >> 4;  // 16-byte groups per quarter (hs <= 128: at most 8)
        const int64_t kg = ((int64_t)kvh * (hs >> 2) + part * per) * seq_len + t;  // group of four elements
        float4 kv[8];
#pragma unroll
        for (int u = 0; u < 8; u++) kv[u] = ldg_nt_f4((const float4 *)kc + kg + (int64_t)(u < per ? u : 0) * seq_len);
        __syncthreads();
#pragma unroll
        for (int u = 0; u < 8; u++) {
            if (u < per) {
                const double k0 = (double)kv[u].x, k1 = (double)kv[u].y, k2 = (double)kv[u].z, k3 = (double)kv[u].w;
#pragma unroll
                for (int g = 0; g < GH; g++) {
                    const double *qq = s_q + g * 128 + 4 * (part * per + u);
                    acc[g] = fma(qq[0], k0, acc[g]);
                    acc[g] = fma(qq[1], k1, acc[g]);
                    acc[g] = fma(qq[2], k2, acc[g]);
                    acc[g] = fma(qq[3], k3, acc[g]);
                }
            }
        }
    }
#pragma unroll
    for (int g = 0; g < GH; g++) s_part[part][g][lane] = acc[g];
    __syncthreads();
    const float scale = sqrtf((float)hs);
    if (threadIdx.x < GH * 64) {  // wavefront g: the 64 scores of head h0 + g, and the largest of them
        const int g = part, l = lane;
        const bool there = t0 + l <= pos;
        const double v = ((s_part[0][g][l] + s_part[1][g][l]) + s_part[2][g][l]) + s_part[3][g][l];
        const float sc = (float)v / scale;
        if (there) att[(int64_t)(h0 + g) * seq_len + t0 + l] = sc;
        const float m = wave_max_f32(there ? sc : -INFINITY);
        if (l == 0) tmax[(int64_t)(h0 + g) * gridDim.x + blockIdx.x] = m;
    }
}

// Softmax over a long cache, first half: a workgroup takes 1024 timesteps of one head.  The head's
// maximum comes from the tiles' maxima; e = fp32(exp(score - max)) replaces the score, the fp64 sum of the
// workgroup's e goes to psum[head][workgroup].  The division by the total is left to the value pass.
__global__ __launch_bounds__(256) void attn_exp_kernel(float *att, const float *tmax, double *psum, const DecodeCtl *ctl,
                                                       int seq_len, int ntiles) {
    __shared__ double redd[4];
    __shared__ float redf[4];
    const int pos = ctl->pos, h = blockIdx.y, c0 = blockIdx.x * 1024;
    if (c0 > pos) return;
    float mx = -INFINITY;
    for (int i = threadIdx.x; i <= pos / 64; i += 256) mx = fmaxf(mx, tmax[(int64_t)h * ntiles + i]);
    mx = block_max_f32(mx, redf);
    float *x = att + (int64_t)h * seq_len;
    double acc = 0.0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int t = c0 + threadIdx.x + 256 * k;
        if (t <= pos) {
            const float e = (float)exp((double)(x[t] - mx));
            x[t] = e;
            acc += (double)e;
        }
    }
    acc = block_sum_f64(acc, redd);
    if (threadIdx.x == 0) psum[(int64_t)h * gridDim.x + blockIdx.x] = acc;
}

// Values: a workgroup = `chunk` (a multiple of 64) timesteps of GH heads sharing a KV head; thread =
// (16-byte group of the head dimension, timestep group), eight loads in flight per round; the
// probabilities p = e / total are formed here (fp32 division, as softmax! does), widened to fp64; fp64
// partial sums per workgroup go to `part`, which attn_reduce4_kernel adds in block order.
template <int GH, bool H16>
__global__ __launch_bounds__(256) void attn_av4_kernel(const float *att, const double *psum, int npsum, const float *vc,
                                                       double *part, const DecodeCtl *ctl, int hs, int n_heads,
                                                       int n_kv_heads, int seq_len, int chunk) {
    __shared__ double s_p[GH][64];
    __shared__ double s_red[8][GH][128];
    const int pos = ctl->pos;
    const int split = blockIdx.x, c0 = split * chunk;
    if (c0 > pos) return;
    const int h0 = blockIdx.y * GH, kvh = h0 / (n_heads / n_kv_heads);
    // the heads' totals: the sums of attn_exp_kernel's workgroups in their order, rounded to fp32 (softmax!'s sum)
    float sf[GH];
#pragma unroll
    for (int g = 0; g < GH; g++) {
        double t = 0.0;
        for (int c = 0; c <= pos / 1024; c++) t += psum[(int64_t)(h0 + g) * npsum + c];
        sf[g] = (float)t;
    }
    if constexpr (H16) {
        // fp16 cache: thread = (16-byte group i8 of eight elements, timestep group tg of 16); a tile of 64 timesteps is
        // four loads per thread, all in flight; the four timestep groups of a wavefront are folded with lane
        // exchanges, the four wavefronts through LDS
        const int n8 = hs >> 3;  // at most 16
        const int i8 = threadIdx.x & 15, tg = threadIdx.x >> 4;
        const bool active = i8 < n8;
        double acc[GH][8];
#pragma unroll
        for (int g = 0; g < GH; g++)
#pragma unroll
            for (int c = 0; c < 8; c++) acc[g][c] = 0.0;
        for (int t0 = c0; t0 < c0 + chunk && t0 <= pos; t0 += 64) {
            const int nt = min(64, pos + 1 - t0);
            __syncthreads();
            for (int i = threadIdx.x; i < GH * 64; i += 256) {
                const int g = i >> 6, l = i & 63;
                float sg = sf[0];
#pragma unroll
                for (int k = 1; k < GH; k++) sg = g == k ? sf[k] : sg;
                s_p[g][l] = l < nt ? (double)(att[(int64_t)(h0 + g) * seq_len + t0 + l] / sg) : 0.0;
            }
            Half8 v[4];
            const int64_t vg = ((int64_t)kvh * seq_len + t0) * n8 + i8;
            h8_bits vb[4];  // (loads first, widening after the last request)
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int l = tg + 16 * u;
                vb[u] = (h8_bits){0u, 0u, 0u, 0u};
                if (active && l < nt) vb[u] = ldg_nt_h8_bits(vc, vg + (int64_t)l * n8);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = h8_widen(vb[u]);
            __syncthreads();
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int l = tg + 16 * u;
#pragma unroll
                for (int g = 0; g < GH; g++) {
                    const double p = s_p[g][l];
#pragma unroll
                    for (int c = 0; c < 8; c++) acc[g][c] = fma(p, (double)v[u].v[c], acc[g][c]);
                }
            }
        }
#pragma unroll
        for (int g = 0; g < GH; g++)
#pragma unroll
            for (int c = 0; c < 8; c++) {
                acc[g][c] += __shfl_xor(acc[g][c], 16, WAVE);
                acc[g][c] += __shfl_xor(acc[g][c], 32, WAVE);
            }
        __syncthreads();
        if (active && (threadIdx.x & 63) < 16) {
#pragma unroll
            for (int g = 0; g < GH; g++)
#pragma unroll
                for (int c = 0; c < 8; c++) s_red[threadIdx.x >> 6][g][8 * i8 + c] = acc[g][c];
        }
        __syncthreads();
        for (int i = threadIdx.x; i < GH * hs; i += 256) {
            const int g = i / hs, e = i % hs;
            double a = 0.0;
            for (int k = 0; k < 4; k++) a += s_red[k][g][e];
            part[((int64_t)split * n_heads + h0 + g) * hs + e] = a;
        }
        return;
    }
    const int n4 = hs >> 2, ngrp = min(8, 256 / n4);  // hs <= 128
    const int i4 = threadIdx.x % n4, tg = threadIdx.x / n4;
    const bool active = tg < ngrp;
    double acc[GH][4];
#pragma unroll
    for (int g = 0; g < GH; g++) acc[g][0] = acc[g][1] = acc[g][2] = acc[g][3] = 0.0;
    for (int t0 = c0; t0 < c0 + chunk && t0 <= pos; t0 += 64) {
        const int nt = min(64, pos + 1 - t0);
        __syncthreads();
        for (int i = threadIdx.x; i < GH * 64; i += 256) {
            const int g = i >> 6, l = i & 63;
            float sg = sf[0];
#pragma unroll
            for (int k = 1; k < GH; k++) sg = g == k ? sf[k] : sg;
            s_p[g][l] = l < nt ? (double)(att[(int64_t)(h0 + g) * seq_len + t0 + l] / sg) : 0.0;
        }
        float4 v[8];
        if (active) {
            const int64_t vg = ((int64_t)kvh * seq_len + t0) * n4 + i4;  // group of four elements
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int l = tg + ngrp * u;
                v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (l < nt) v[u] = ldg_nt_f4((const float4 *)vc + vg + (int64_t)l * n4);
            }
        }
        __syncthreads();
        if (active) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int l = tg + ngrp * u;
                if (l < 64) {
#pragma unroll
                    for (int g = 0; g < GH; g++) {
                        const double p = s_p[g][l];
                        acc[g][0] = fma(p, (double)v[u].x, acc[g][0]);
                        acc[g][1] = fma(p, (double)v[u].y, acc[g][1]);
                        acc[g][2] = fma(p, (double)v[u].z, acc[g][2]);
                        acc[g][3] = fma(p, (double)v[u].w, acc[g][3]);
                    }
                }
            }
        }
    }
    if (active) {
#pragma unroll
        for (int g = 0; g < GH; g++)
#pragma unroll
            for (int c = 0; c < 4; c++) s_red[tg][g][4 * i4 + c] = acc[g][c];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < GH * hs; i += 256) {
        const int g = i / hs, e = i % hs;
        double a = 0.0;
        for (int k = 0; k < ngrp; k++) a += s_red[k][g][e];
        part[((int64_t)split * n_heads + h0 + g) * hs + e] = a;
    }
}

// out[e] = fp32(sum of the partial sums of the timestep blocks, in block order): 64 elements per
// workgroup, four threads per element each adding a quarter of the blocks, quarters added in order
__global__ __launch_bounds__(256) void attn_reduce4_kernel(const double *part, float *out, const DecodeCtl *ctl,
                                                           int dim, int chunk) {
    __shared__ double s_q[4][64];
    const int e = blockIdx.x * 64 + (threadIdx.x & 63), qtr = threadIdx.x >> 6;
    const int nsplit = ctl->pos / chunk + 1;
    const int per = (nsplit + 3) >> 2;
    double acc = 0.0;
    if (e < dim) {
        const int s1 = min(nsplit, (qtr + 1) * per);
#pragma unroll 8
        for (int s = qtr * per; s < s1; s++) acc += part[(int64_t)s * dim + e];
    }
    s_q[qtr][threadIdx.x & 63] = acc;
    __syncthreads();
    if (qtr == 0 && e < dim) out[e] = (float)(((s_q[0][threadIdx.x] + s_q[1][threadIdx.x]) + s_q[2][threadIdx.x]) + s_q[3][threadIdx.x]);
}

// Short sequences: one workgroup per head does scores, softmax and values in one launch.
__global__ __launch_bounds__(1024) void attn_fused_kernel(const float *q, float *xb, const float *kc, const float *vc,
                                                          const DecodeCtl *ctl, int hs, int n_heads, int n_kv_heads,
                                                          int seq_len) {
    extern __shared__ uint4 smem[];
    __shared__ double redd[16];
    __shared__ float redf[16];
    attention_head<false>(q, xb, kc, vc, hs, n_heads, n_kv_heads, seq_len, blockIdx.x, ctl->pos, smem, redd, redf);
}

hipError_t k_attention_fused(hipStream_t s, const float *q, float *xb, const float *kc, const float *vc,
                             const DecodeCtl *ctl, int head_size, int n_heads, int n_kv_heads, int seq_len) {
    const size_t lds = (size_t)head_size * 8 + (size_t)seq_len * 8 + (size_t)(1024 / head_size) * head_size * 8 +
                       (size_t)seq_len * 4;
    if (lds > 64 * 1024) return hipErrorInvalidValue;
    hipLaunchKernelGGL(attn_fused_kernel, dim3(n_heads), dim3(1024), lds, s, q, xb, kc, vc, ctl, head_size, n_heads,
                       n_kv_heads, seq_len);
    return hipGetLastError();
}

template <int GH, bool H16>
static hipError_t launch_attn(hipStream_t s, const double *qd, const float *kc, const float *vc, float *att,
                              double *pd, double *part, float *out, const DecodeCtl *ctl, int hs,
                              int n_heads, int n_kv_heads, int seq_len) {
    const int ntiles = (seq_len + L2H_ATT_TILE - 1) / L2H_ATT_TILE;
    if (hs <= 128 && hs % 16 == 0 && L2H_ATT_TILE == 64) {
        // (pd, seq_len doubles per head, holds the softmax workgroups' sums and after them the tiles' maxima)
        const int npsum = (seq_len + 1023) / 1024;
        double *psum = pd;
        float *tmax = (float *)(pd + (int64_t)n_heads * npsum);
        hipLaunchKernelGGL((attn_scores4_kernel<GH, H16>), dim3(ntiles, n_heads / GH), dim3(256), 0, s, qd, kc, att, tmax, ctl,
                           hs, n_heads, n_kv_heads, seq_len);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(attn_exp_kernel, dim3(npsum, n_heads), dim3(256), 0, s, att, tmax, psum, ctl, seq_len, ntiles);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
        // timesteps per value workgroup: as large as still leaves L2H_AV_MIN_WGS workgroups over a full cache
        int chunk = 64;
        while (chunk < 512 && (int64_t)(seq_len / (2 * chunk)) * (n_heads / GH) >= L2H_AV_MIN_WGS) chunk *= 2;
        hipLaunchKernelGGL((attn_av4_kernel<GH, H16>), dim3((seq_len + chunk - 1) / chunk, n_heads / GH), dim3(256), 0, s, att,
                           psum, npsum, vc, part, ctl, hs, n_heads, n_kv_heads, seq_len, chunk);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
        const int dim = hs * n_heads;
        hipLaunchKernelGGL(attn_reduce4_kernel, dim3((dim + 63) / 64), dim3(256), 0, s, part, out, ctl, dim, chunk);
        return hipGetLastError();
    }
    if (H16) return hipErrorInvalidValue;  // (the general kernels below read fp32 caches only)
    hipLaunchKernelGGL((attn_scores_kernel<GH>), dim3((ntiles + 3) / 4, n_heads / GH), dim3(256), 0, s, qd, kc, att,
                       ctl, hs, n_heads, n_kv_heads, seq_len);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(attn_softmax_kernel, dim3(n_heads), dim3(256), 0, s, att, pd, ctl, seq_len);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((attn_av_kernel<GH>), dim3(ntiles, n_heads / GH), dim3(hs), 0, s, pd, vc, part, ctl, hs,
                       n_heads, n_kv_heads, seq_len);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int dim = hs * n_heads;
    hipLaunchKernelGGL(attn_reduce_kernel, dim3((dim + 255) / 256), dim3(256), 0, s, part, out, ctl, dim);
    return hipGetLastError();
}

hipError_t k_attention(hipStream_t s, const double *qd, const float *kc, const float *vc, float *att, double *pd,
                       double *part, float *out, const DecodeCtl *ctl, int head_size, int n_heads,
                       int n_kv_heads, int seq_len, int kv16) {
    const int G = n_heads / n_kv_heads;
#define GO(GH_)                                                                                                          \
    return kv16 ? launch_attn<GH_, true>(s, qd, kc, vc, att, pd, part, out, ctl, head_size, n_heads, n_kv_heads, seq_len) \
                : launch_attn<GH_, false>(s, qd, kc, vc, att, pd, part, out, ctl, head_size, n_heads, n_kv_heads, seq_len)
    if (G % 4 == 0) GO(4);
    if (G % 2 == 0) GO(2);
    GO(1);
#undef GO
}

// Decode attention for one position (reference src/inference.jl:176-220, 263-278):
//   scores   att[h][t] = fp32(sum_fp64 q[h][i]*K[t][i]) / sqrt(hs)      attention_weights!, :268
//   softmax  per head: max, exp (fp64, rounded to fp32), fp64 sum, p = e / sum   softmax!
//   values   out[h][i] = fp32(sum_fp64 p[h][t]*V[t][i])                 combine_values!
// Grids are sized for seq_len and exit early past the current position, so one recorded
// launch sequence serves every position.
// K cache layout per layer: [n_kv_heads][hs/4][seq_len][4] (a lane per timestep reads
// contiguous 16-byte pieces); V cache: [n_kv_heads][seq_len][hs] (a lane per feature).
#include "matvec_dev.h"

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
__global__ __launch_bounds__(256) void attn_softmax_kernel(float *att, double *pd, const DecodeCtl *ctl, int seq_len) {
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

template <int GH>
static hipError_t launch_attn(hipStream_t s, const double *qd, const float *kc, const float *vc, float *att,
                              double *pd, double *part, float *out, const DecodeCtl *ctl, int hs, int n_heads,
                              int n_kv_heads, int seq_len) {
    const int ntiles = (seq_len + L2H_ATT_TILE - 1) / L2H_ATT_TILE;
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
                       double *part, float *out, const DecodeCtl *ctl, int head_size, int n_heads, int n_kv_heads,
                       int seq_len) {
    const int G = n_heads / n_kv_heads;
    if (G % 4 == 0) return launch_attn<4>(s, qd, kc, vc, att, pd, part, out, ctl, head_size, n_heads, n_kv_heads, seq_len);
    if (G % 2 == 0) return launch_attn<2>(s, qd, kc, vc, att, pd, part, out, ctl, head_size, n_heads, n_kv_heads, seq_len);
    return launch_attn<1>(s, qd, kc, vc, att, pd, part, out, ctl, head_size, n_heads, n_kv_heads, seq_len);
}

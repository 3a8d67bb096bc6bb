// Device-side helpers shared by the kernel files (gfx950, wavefront = 64 lanes).
#pragma once

#include "l2h_internal.h"

#define WAVE 64

__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

// index of element i of head kvh at timestep t in the fp16 K cache
__device__ __forceinline__ int64_t kc16_index(int kvh, int i, int t, int hs, int seq_len) {
    return (((int64_t)kvh * (hs >> 3) + (i >> 3)) * seq_len + t) * 8 + (i & 7);
}

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, WAVE);
    return v;
}

__device__ __forceinline__ float wave_max_f32(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, WAVE));
    return v;
}

// Sum of one double per thread over a workgroup of up to 1024 threads; every thread gets
// the total.  `red` is LDS scratch of at least 16 doubles.  The order of the fp64
// additions is fixed by the thread layout.
__device__ __forceinline__ double block_sum_f64(double v, double *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum_f64(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    double t = 0.0;
    for (int w = 0; w < nw; w++) t += red[w];
    return t;
}

__device__ __forceinline__ float block_max_f32(float v, float *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_max_f32(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int w = 1; w < nw; w++) t = fmaxf(t, red[w]);
    return t;
}

// 6-bit scale/min pairs of sub-blocks 2j and 2j+1 from a q4_K/q5_K header
// (hdr.x = d | dmin<<16, hdr.y/z/w = the 12 packed scale bytes).
// Follows the unpacking in src/kquants.jl:80-81,86-87 (sub-blocks 0..3) and
// :102-103,108-109 (sub-blocks 4..7) of the reference.
__device__ __forceinline__ void kq_scales_pair(const uint4 hdr, int j, int &sc_a, int &sc_b, int &m_a, int &m_b) {
    const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
    const int sh = 16 * (j & 1);
    const uint32_t a0 = s0 >> sh, a1 = s1 >> sh, a2 = s2 >> sh;
    if (j < 2) {
        sc_a = a0 & 63;
        sc_b = (a0 >> 8) & 63;
        m_a = a1 & 63;
        m_b = (a1 >> 8) & 63;
    } else {
        sc_a = (a2 & 0xF) | (((a0 >> 6) & 3) << 4);
        m_a = ((a2 >> 4) & 0xF) | (((a1 >> 6) & 3) << 4);
        sc_b = ((a2 >> 8) & 0xF) | (((a0 >> 14) & 3) << 4);
        m_b = ((a2 >> 12) & 0xF) | (((a1 >> 14) & 3) << 4);
    }
}

// scale/min of a single sub-block s (0..7)
__device__ __forceinline__ void kq_scale_min(const uint4 hdr, int s, int &sc, int &m) {
    int sa, sb, ma, mb;
    kq_scales_pair(hdr, s >> 1, sa, sb, ma, mb);
    sc = (s & 1) ? sb : sa;
    m = (s & 1) ? mb : ma;
}

// Weight value of element e (0..ne0) of row `row`, formed with the reference's fp32
// expressions (src/kquants.jl:93,97 q4_K; :213,217 q5_K; :340-343 q6_K).
__device__ __forceinline__ float dequant_elem(const DevTensor &t, int64_t row, int64_t e) {
    if (t.type == L2H_TYPE_F32) return t.f32[row * t.ne0 + e];
    const int64_t blk = row * t.nb + (e >> 8);
    const int r = (int)(e & 255);
    if (t.type == L2H_TYPE_Q4_K || t.type == L2H_TYPE_Q5_K) {
        const uint4 hdr = t.hdr[blk];
        const float d = half_bits_to_float((uint16_t)(hdr.x & 0xFFFF));
        const float dmin = half_bits_to_float((uint16_t)(hdr.x >> 16));
        const int s = r >> 5, j = r >> 6, l = r & 31;
        int sc, m;
        kq_scale_min(hdr, s, sc, m);
        const uint8_t byte = t.qs[blk * 128 + 32 * j + l];
        int q = (s & 1) ? (byte >> 4) : (byte & 0xF);
        if (t.type == L2H_TYPE_Q5_K) {
            const uint8_t hb = t.qh[blk * 32 + l];
            if (hb & (1u << s)) q += 16;
        }
        const float d1 = d * (float)sc, m1 = dmin * (float)m;
        return d1 * (float)q - m1;
    }
    // Q6_K
    const int n = r >> 7, rr = r & 127, g = rr >> 5, l = rr & 31;
    const uint8_t lo = t.qs[blk * 128 + 64 * n + l + ((g & 1) ? 32 : 0)];
    const uint8_t hb = t.qh[blk * 64 + 32 * n + l];
    const int nib = (g & 2) ? (lo >> 4) : (lo & 0xF);
    const int q = (nib | (((hb >> (2 * g)) & 3) << 4)) - 32;
    const int hh = l >> 4;
    const uint32_t scw = t.sc6[blk * 4 + 2 * n + hh];
    const int sc = (int)(int8_t)((scw >> (8 * g)) & 0xFF);
    const float d = half_bits_to_float(t.d6[blk]);
    return d * (float)(sc * q);
}

// matmul!(y, A, x) for one input vector (reference src/matmul.jl:3-23):
//   k-quant weights x q8_K activations -> integer dot products (packed-int8 dot
//   instructions on nibbles unpacked in registers), scaled and summed in fp64;
//   F32 weights x fp32 activations -> fp64 sum of exact products.
// Every output row is   fp32( sum over super-blocks of exact fp64 terms ),   so the result
// does not depend on how lanes and wavefronts split the row.
#include "dev_common.h"

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// Activations staged in LDS for one workgroup.
struct XLds {
    const int8_t *qs;
    const int16_t *bsums;
    const float *d;
};

// ---- per-lane chunk kernels ------------------------------------------------------------------
// q4_K: lane chunk c (0..7) of a block = qs bytes [16c, 16c+16): low nibbles are elements
// 64j+16h+k of sub-block 2j, high nibbles elements 64j+32+16h+k of sub-block 2j+1
// (j = c>>1, h = c&1; reference src/kquants.jl:92-98).
__device__ __forceinline__ void chunk_q4k(const uint4 w, const uint4 hdr, int c, const XLds &x, int64_t blk_in_row,
                                          int &i_sc, int &i_min) {
    const int j = c >> 1, h = c & 1;
    int sc_a, sc_b, m_a, m_b;
    kq_scales_pair(hdr, j, sc_a, sc_b, m_a, m_b);
    const int8_t *xb = x.qs + blk_in_row * 256 + 64 * j + 16 * h;
    const uint4 xlo = *(const uint4 *)xb;
    const uint4 xhi = *(const uint4 *)(xb + 32);
    int dot_a = 0, dot_b = 0;
    dot_a = sdot4(w.x & 0x0F0F0F0Fu, xlo.x, dot_a);
    dot_a = sdot4(w.y & 0x0F0F0F0Fu, xlo.y, dot_a);
    dot_a = sdot4(w.z & 0x0F0F0F0Fu, xlo.z, dot_a);
    dot_a = sdot4(w.w & 0x0F0F0F0Fu, xlo.w, dot_a);
    dot_b = sdot4((w.x >> 4) & 0x0F0F0F0Fu, xhi.x, dot_b);
    dot_b = sdot4((w.y >> 4) & 0x0F0F0F0Fu, xhi.y, dot_b);
    dot_b = sdot4((w.z >> 4) & 0x0F0F0F0Fu, xhi.z, dot_b);
    dot_b = sdot4((w.w >> 4) & 0x0F0F0F0Fu, xhi.w, dot_b);
    const int16_t *bs = x.bsums + blk_in_row * 16 + 4 * j + h;
    i_sc = sc_a * dot_a + sc_b * dot_b;
    i_min = m_a * (int)bs[0] + m_b * (int)bs[2];
}

// q5_K: as q4_K plus the fifth bit: bit 2j of qh[l] for the low-nibble element, bit 2j+1
// for the high-nibble element, l = 16h+k (reference src/kquants.jl:213,217,220-221).
__device__ __forceinline__ void chunk_q5k(const uint4 w, const uint4 qh, const uint4 hdr, int c, const XLds &x,
                                          int64_t blk_in_row, int &i_sc, int &i_min) {
    const int j = c >> 1, h = c & 1;
    int sc_a, sc_b, m_a, m_b;
    kq_scales_pair(hdr, j, sc_a, sc_b, m_a, m_b);
    const int8_t *xb = x.qs + blk_in_row * 256 + 64 * j + 16 * h;
    const uint4 xlo = *(const uint4 *)xb;
    const uint4 xhi = *(const uint4 *)(xb + 32);
    const int sa = 2 * j, sb = 2 * j + 1;
    int dot_a = 0, dot_b = 0;
#define Q5LO(W, H) (((W)&0x0F0F0F0Fu) | ((((H) >> sa) & 0x01010101u) << 4))
#define Q5HI(W, H) ((((W) >> 4) & 0x0F0F0F0Fu) | ((((H) >> sb) & 0x01010101u) << 4))
    dot_a = sdot4(Q5LO(w.x, qh.x), xlo.x, dot_a);
    dot_a = sdot4(Q5LO(w.y, qh.y), xlo.y, dot_a);
    dot_a = sdot4(Q5LO(w.z, qh.z), xlo.z, dot_a);
    dot_a = sdot4(Q5LO(w.w, qh.w), xlo.w, dot_a);
    dot_b = sdot4(Q5HI(w.x, qh.x), xhi.x, dot_b);
    dot_b = sdot4(Q5HI(w.y, qh.y), xhi.y, dot_b);
    dot_b = sdot4(Q5HI(w.z, qh.z), xhi.z, dot_b);
    dot_b = sdot4(Q5HI(w.w, qh.w), xhi.w, dot_b);
#undef Q5LO
#undef Q5HI
    const int16_t *bs = x.bsums + blk_in_row * 16 + 4 * j + h;
    i_sc = sc_a * dot_a + sc_b * dot_b;
    i_min = m_a * (int)bs[0] + m_b * (int)bs[2];
}

// q6_K: lane chunk c (0..3) of a block = ql bytes [64n+16h, +16) and [64n+32+16h, +16)
// with qh bytes [32n+16h, +16), n = c>>1, h = c&1: four groups of 16 elements at
// 128n + 32g + 16h, g = 0..3 (reference src/kquants.jl:333-343).  q-32 is folded in through
// the q8_K group sums: sum (q-32)*x = sum q*x - 32*bsum.
__device__ __forceinline__ int chunk_q6k(const uint4 la, const uint4 lb, const uint4 qh, uint32_t scw, int c,
                                         const XLds &x, int64_t blk_in_row) {
    const int n = c >> 1, h = c & 1;
    const int8_t *xb = x.qs + blk_in_row * 256 + 128 * n + 16 * h;
    const uint4 x0 = *(const uint4 *)xb, x1 = *(const uint4 *)(xb + 32), x2 = *(const uint4 *)(xb + 64),
                x3 = *(const uint4 *)(xb + 96);
    int d0 = 0, d1 = 0, d2 = 0, d3 = 0;
#define Q6STEP(A, B, H, X0, X1, X2, X3)                                           \
    d0 = sdot4(((A)&0x0F0F0F0Fu) | (((H) << 4) & 0x30303030u), X0, d0);           \
    d1 = sdot4(((B)&0x0F0F0F0Fu) | (((H) << 2) & 0x30303030u), X1, d1);           \
    d2 = sdot4((((A) >> 4) & 0x0F0F0F0Fu) | ((H)&0x30303030u), X2, d2);           \
    d3 = sdot4((((B) >> 4) & 0x0F0F0F0Fu) | (((H) >> 2) & 0x30303030u), X3, d3);
    Q6STEP(la.x, lb.x, qh.x, x0.x, x1.x, x2.x, x3.x)
    Q6STEP(la.y, lb.y, qh.y, x0.y, x1.y, x2.y, x3.y)
    Q6STEP(la.z, lb.z, qh.z, x0.z, x1.z, x2.z, x3.z)
    Q6STEP(la.w, lb.w, qh.w, x0.w, x1.w, x2.w, x3.w)
#undef Q6STEP
    const int16_t *bs = x.bsums + blk_in_row * 16 + 8 * n + h;
    const int s0 = (int)(int8_t)(scw & 0xFF), s1 = (int)(int8_t)((scw >> 8) & 0xFF),
              s2 = (int)(int8_t)((scw >> 16) & 0xFF), s3 = (int)(int8_t)(scw >> 24);
    return s0 * (d0 - 32 * (int)bs[0]) + s1 * (d1 - 32 * (int)bs[2]) + s2 * (d2 - 32 * (int)bs[4]) +
           s3 * (d3 - 32 * (int)bs[6]);
}

// ---- one row of one k-quant tensor against the staged activations; returns this lane's
// share of the row sum (fp64).  DEBUG also stores the per-block integer sums.
template <int TYPE, bool DEBUG>
__device__ __forceinline__ double row_partial(const DevTensor &w, int64_t row, const XLds &x, int lane,
                                              int32_t *dbg_isc, int32_t *dbg_imin, int64_t dbg_row) {
    const int64_t nb = w.nb;
    double acc = 0.0;
    if (TYPE == L2H_TYPE_Q6_K) {
        const int nchunks = (int)nb * 4;
        const uint4 *ql = (const uint4 *)w.qs + row * nb * 8;
        const uint4 *qh = (const uint4 *)w.qh + row * nb * 4;
        const uint32_t *sc = w.sc6 + row * nb * 4;
        const uint16_t *dd = w.d6 + row * nb;
        for (int g = lane; g < nchunks; g += WAVE) {
            const int b = g >> 2, c = g & 3, n = c >> 1, h = c & 1;
            const uint4 la = ql[b * 8 + 4 * n + h];
            const uint4 lb = ql[b * 8 + 4 * n + 2 + h];
            const uint4 hv = qh[b * 4 + 2 * n + h];
            const uint32_t scw = sc[b * 4 + 2 * n + h];
            const float d = half_bits_to_float(dd[b]);
            int i_sc = chunk_q6k(la, lb, hv, scw, c, x, b);
            const float dy = d * x.d[b];
            acc = fma((double)dy, (double)i_sc, acc);
            if (DEBUG) {
                i_sc += __shfl_xor(i_sc, 1, WAVE);
                i_sc += __shfl_xor(i_sc, 2, WAVE);
                if (c == 0) {
                    dbg_isc[dbg_row * nb + b] = i_sc;
                    dbg_imin[dbg_row * nb + b] = 0;
                }
            }
        }
    } else {
        const int nchunks = (int)nb * 8;
        const uint4 *qs = (const uint4 *)w.qs + row * nb * 8;
        const uint4 *hd = w.hdr + row * nb;
        const uint4 *qh = (const uint4 *)w.qh + row * nb * 2;
        for (int g = lane; g < nchunks; g += WAVE) {
            const int b = g >> 3, c = g & 7;
            const uint4 wv = qs[g];
            const uint4 hdr = hd[b];
            int i_sc, i_min;
            if (TYPE == L2H_TYPE_Q5_K) {
                const uint4 hv = qh[b * 2 + (c & 1)];
                chunk_q5k(wv, hv, hdr, c, x, b, i_sc, i_min);
            } else {
                chunk_q4k(wv, hdr, c, x, b, i_sc, i_min);
            }
            const float yd = x.d[b];
            const float dy = half_bits_to_float((uint16_t)(hdr.x & 0xFFFF)) * yd;
            const float my = half_bits_to_float((uint16_t)(hdr.x >> 16)) * yd;
            acc = fma((double)dy, (double)i_sc, acc);
            acc = fma(-(double)my, (double)i_min, acc);
            if (DEBUG) {
                i_sc += __shfl_xor(i_sc, 1, WAVE);
                i_min += __shfl_xor(i_min, 1, WAVE);
                i_sc += __shfl_xor(i_sc, 2, WAVE);
                i_min += __shfl_xor(i_min, 2, WAVE);
                i_sc += __shfl_xor(i_sc, 4, WAVE);
                i_min += __shfl_xor(i_min, 4, WAVE);
                if (c == 0) {
                    dbg_isc[dbg_row * nb + b] = i_sc;
                    dbg_imin[dbg_row * nb + b] = i_min;
                }
            }
        }
    }
    return acc;
}

// Rows per wavefront pass: their loads are issued together to keep HBM requests in flight.
#define MV_R 4

template <int TYPE, bool DEBUG>
__global__ __launch_bounds__(256) void matvec_kq_kernel(MatvecArgs a) {
    extern __shared__ uint4 smem[];
    const int64_t K = a.seg[0].w.ne0;
    int8_t *s_qs = (int8_t *)smem;
    int16_t *s_bs = (int16_t *)(s_qs + K);
    float *s_d = (float *)(s_qs + K + K / 8);
    {
        const uint4 *g_qs = (const uint4 *)a.xq.qs;
        for (int i = threadIdx.x; i < K / 16; i += blockDim.x) ((uint4 *)s_qs)[i] = g_qs[i];
        const uint4 *g_bs = (const uint4 *)a.xq.bsums;
        for (int i = threadIdx.x; i < K / 128; i += blockDim.x) ((uint4 *)s_bs)[i] = g_bs[i];
        for (int i = threadIdx.x; i < K / 256; i += blockDim.x) s_d[i] = a.xq.d[i];
    }
    __syncthreads();
    XLds x{s_qs, s_bs, s_d};

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    for (int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * MV_R; row0 < a.total_rows; row0 += nwaves * MV_R) {
        double acc[MV_R];
#pragma unroll
        for (int r = 0; r < MV_R; r++) {
            acc[r] = 0.0;
            int64_t row = row0 + r;
            if (row < a.total_rows) {
                int sidx = 0;
                if (a.nseg > 1 && row >= a.seg[0].w.ne1) {
                    row -= a.seg[0].w.ne1;
                    sidx = 1;
                    if (a.nseg > 2 && row >= a.seg[1].w.ne1) {
                        row -= a.seg[1].w.ne1;
                        sidx = 2;
                    }
                }
                acc[r] = row_partial<TYPE, DEBUG>(a.seg[sidx].w, row, x, lane, a.dbg_isc, a.dbg_imin, row0 + r);
            }
        }
#pragma unroll
        for (int r = 0; r < MV_R; r++) acc[r] = wave_sum_f64(acc[r]);
        if (lane < MV_R) {
            double v = acc[0];
#pragma unroll
            for (int r = 1; r < MV_R; r++)
                if (lane == r) v = acc[r];
            int64_t row = row0 + lane;
            if (row < a.total_rows) {
                int sidx = 0;
                if (a.nseg > 1 && row >= a.seg[0].w.ne1) {
                    row -= a.seg[0].w.ne1;
                    sidx = 1;
                    if (a.nseg > 2 && row >= a.seg[1].w.ne1) {
                        row -= a.seg[1].w.ne1;
                        sidx = 2;
                    }
                }
                float res = (float)v;
                if (a.resid) res = a.resid[row] + res;
                a.seg[sidx].y[row] = res;
            }
        }
    }
}

// F32 weights: y[row] = fp32( sum_fp64 A[row][k] * x[k] )
__global__ __launch_bounds__(256) void matvec_f32_kernel(MatvecArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    const int64_t K = a.seg[0].w.ne0;
    for (int64_t grow = (int64_t)blockIdx.x * 4 + wave; grow < a.total_rows; grow += nwaves) {
        int64_t row = grow;
        int sidx = 0;
        if (a.nseg > 1 && row >= a.seg[0].w.ne1) {
            row -= a.seg[0].w.ne1;
            sidx = 1;
            if (a.nseg > 2 && row >= a.seg[1].w.ne1) {
                row -= a.seg[1].w.ne1;
                sidx = 2;
            }
        }
        const float *wr = a.seg[sidx].w.f32 + row * K;
        double acc = 0.0;
        if ((K & 3) == 0) {
            const float4 *w4 = (const float4 *)wr;
            const float4 *x4 = (const float4 *)a.xf;
            for (int64_t i = lane; i < K / 4; i += WAVE) {
                const float4 wv = w4[i], xv = x4[i];
                acc = fma((double)wv.x, (double)xv.x, acc);
                acc = fma((double)wv.y, (double)xv.y, acc);
                acc = fma((double)wv.z, (double)xv.z, acc);
                acc = fma((double)wv.w, (double)xv.w, acc);
            }
        } else {
            for (int64_t i = lane; i < K; i += WAVE) acc = fma((double)wr[i], (double)a.xf[i], acc);
        }
        acc = wave_sum_f64(acc);
        if (lane == 0) {
            float res = (float)acc;
            if (a.resid) res = a.resid[row] + res;
            a.seg[sidx].y[row] = res;
        }
    }
}

template <int TYPE>
static hipError_t launch_kq(hipStream_t s, const MatvecArgs &a) {
    const int64_t K = a.seg[0].w.ne0;
    const size_t lds = (size_t)(K + K / 8 + K / 64);
    int64_t grid = (a.total_rows + 4 * MV_R - 1) / (4 * MV_R);
    if (grid > 256 * 8) grid = 256 * 8;
    if (a.dbg_isc)
        hipLaunchKernelGGL((matvec_kq_kernel<TYPE, true>), dim3((unsigned)grid), dim3(256), lds, s, a);
    else
        hipLaunchKernelGGL((matvec_kq_kernel<TYPE, false>), dim3((unsigned)grid), dim3(256), lds, s, a);
    return hipGetLastError();
}

hipError_t k_matvec(hipStream_t s, const MatvecArgs &a) {
    const int type = a.seg[0].w.type;
    switch (type) {
    case L2H_TYPE_Q4_K: return launch_kq<L2H_TYPE_Q4_K>(s, a);
    case L2H_TYPE_Q5_K: return launch_kq<L2H_TYPE_Q5_K>(s, a);
    case L2H_TYPE_Q6_K: return launch_kq<L2H_TYPE_Q6_K>(s, a);
    case L2H_TYPE_F32: {
        int64_t grid = (a.total_rows + 3) / 4;
        if (grid > 256 * 8) grid = 256 * 8;
        hipLaunchKernelGGL(matvec_f32_kernel, dim3((unsigned)grid), dim3(256), 0, s, a);
        return hipGetLastError();
    }
    }
    return hipErrorInvalidValue;
}
